// extern "C" entry points of libmsd_hip.so: argument checks, then dispatch to
// the kernels.  Nothing here touches the device before the checks pass, so
// every MSD_ERR_INVALID path can be exercised on a machine without a GPU.
#include "../../include/msd_hip.h"
#include "msd_kernels.h"

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

namespace msd {
const char *const kKnobNames[kKnobCount] = {
    "bwdx.vec2d", "bwdx.vec3d", "bwdx.unroll2d", "bwdx.unroll3d", "bwdx.min_blocks",
    "xcd_remap", "bwdk.vec2d", "bwdk.vec3d", "bwdk.blocks",
    "fwd.vec2d", "fwd.vec3d", "fwd.split", "fwd.rows2d", "bwdk.rows", "block.fuse",
    "block.defer", "bwdk.interleave", "block.snake", "fwd.class3d", "fwd.lattice3d",
    "block.pair", "block.triple", "final.tiled", "block.split3d", "block.chainpair", "bwdk.fused3d", "bwdx.lean1",
};
static_assert(kKnobBwdxLean1 + 1 == kKnobCount, "one name per knob, in the order of the enum");
int g_knobs[kKnobCount];
// every knob starts at "library default"
const bool g_knobs_ready = [] {
    for (int i = 0; i < kKnobCount; i++) g_knobs[i] = -1;
    return true;
}();
int knob(Knob k, int dflt) { return g_knobs[k] < 0 ? dflt : g_knobs[k]; }
}  // namespace msd

namespace {

thread_local std::string g_error;

// 0: specialised kernels where they apply (default); 1: shape-generic kernels only.
int g_kernel_path = 0;

template <typename T> struct is_f32 { static constexpr bool value = false; };
template <> struct is_f32<float> { static constexpr bool value = true; };

// Optional per-class kernel timing with HIP events recorded on the launch stream
// (msd_profile_* in the C ABI).
constexpr int kProfileClasses = 4;   // forward, backward_x (+ mask), backward_k(+bias), fused backward_x+k

struct Profile {
    bool on = false;
    std::vector<hipEvent_t> pool;                           // reused across calls
    size_t used = 0;
    struct Span {
        size_t start, stop;                                  // indices into pool
        int64_t calls;                                       // operator calls the span covers
    };
    std::vector<Span> spans[kProfileClasses];
    // Inside a block loop (ProfileBatch) consecutive launches of one class share ONE pair of
    // events, and the event that ends a run starts the next one: a pair per launch costs about
    // four microseconds of idle stream per launch, which would be charged to the kernels.
    bool batching = false;
    int open_cls = -1;
    size_t open_start = 0;
    int64_t open_calls = 0;

    // index of a fresh event recorded on s, or SIZE_MAX
    size_t record(hipStream_t s)
    {
        if (used == pool.size()) {
            hipEvent_t e;
            if (hipEventCreate(&e) != hipSuccess) return SIZE_MAX;
            pool.push_back(e);
        }
        if (hipEventRecord(pool[used], s) != hipSuccess) return SIZE_MAX;
        return used++;
    }
    // ends the open run of a batch (if any) at a new event and returns that event's index
    size_t close_run(hipStream_t s)
    {
        const size_t e = record(s);
        if (open_cls >= 0 && e != SIZE_MAX) spans[open_cls].push_back({open_start, e, open_calls});
        open_cls = -1;
        return e;
    }
} g_profile;

// Records an event pair around the launches made during its lifetime.  `counted` false:
// the time is added to the class, the number of calls is not (work done on behalf of calls
// that were counted already).
struct ProfileScope {
    int cls;
    hipStream_t s;
    size_t start = 0;
    bool active;
    int64_t calls;
    ProfileScope(int cls_, hipStream_t s_, bool counted = true)
        : cls(cls_), s(s_), active(g_profile.on), calls(counted ? 1 : 0)
    {
        if (!active) return;
        if (g_profile.batching) {
            active = false;                       // the run's events do the timing
            if (g_profile.open_cls != cls) {
                const size_t e = g_profile.close_run(s);
                if (e == SIZE_MAX) return;
                g_profile.open_cls = cls;
                g_profile.open_start = e;
                g_profile.open_calls = 0;
            }
            g_profile.open_calls += calls;
            return;
        }
        start = g_profile.record(s);
        if (start == SIZE_MAX) active = false;
    }
    ~ProfileScope()
    {
        if (!active) return;
        const size_t stop = g_profile.record(s);
        if (stop != SIZE_MAX) g_profile.spans[cls].push_back({start, stop, calls});
    }
};

// For the lifetime of this object the scopes on stream s are merged into runs per class.
struct ProfileBatch {
    hipStream_t s;
    bool active;
    explicit ProfileBatch(hipStream_t s_) : s(s_), active(g_profile.on && !g_profile.batching)
    {
        if (!active) return;
        g_profile.batching = true;
        g_profile.open_cls = -1;
    }
    ~ProfileBatch()
    {
        if (!active) return;
        if (g_profile.open_cls >= 0) g_profile.close_run(s);
        g_profile.batching = false;
    }
};

int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

int hip_fail(const char *where, hipError_t e)
{
    return fail(MSD_ERR_HIP, "%s: %s", where, hipGetErrorString(e));
}

// Geometry checks shared by all operators (rank, extents, dilation rule of
// msd_custom_convolutions.cpp:39-52).  c_in may be 0 for the bias-only ops.
int make_geom(const char *fn, int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
              const int64_t *spatial, int dilation, bool need_dilation, msd::Geom *g)
{
    if (dtype != MSD_F32 && dtype != MSD_F64) return fail(MSD_ERR_INVALID, "%s: dtype must be MSD_F32 or MSD_F64", fn);
    if (ndim != 2 && ndim != 3) return fail(MSD_ERR_INVALID, "%s: expected 2 or 3 spatial dimensions, got %d", fn, ndim);
    if (!spatial) return fail(MSD_ERR_INVALID, "%s: spatial is NULL", fn);
    if (batch <= 0 || c_in < 0 || c_out <= 0)
        return fail(MSD_ERR_INVALID, "%s: batch and channel counts must be positive", fn);
    int64_t nvox = 1;
    for (int i = 0; i < ndim; i++) {
        if (spatial[i] <= 0) return fail(MSD_ERR_INVALID, "%s: spatial extents must be positive", fn);
        nvox *= spatial[i];
        if (nvox >= (int64_t(1) << 30)) return fail(MSD_ERR_INVALID, "%s: more than 2^30 voxels per channel", fn);
    }
    if (batch > 65535) return fail(MSD_ERR_INVALID, "%s: batch larger than 65535", fn);
    if (c_in >= (1 << 20) || c_out >= (1 << 16)) return fail(MSD_ERR_INVALID, "%s: channel count too large", fn);
    if (need_dilation) {
        if (dilation <= 0) return fail(MSD_ERR_INVALID, "%s: Dilation must be 1 or greater", fn);
        for (int i = 0; i < ndim; i++)
            if (dilation > spatial[i])
                return fail(MSD_ERR_INVALID, "%s: Dilation cannot be greater than size of image.", fn);
    }
    g->ndim = ndim;
    g->reverse = 0;
    g->B = (int)batch;
    g->C = (int)c_in;
    g->Wd = (int)c_out;
    g->D = ndim == 3 ? (int)spatial[0] : 1;
    g->H = (int)spatial[ndim - 2];
    g->W = (int)spatial[ndim - 1];
    g->dil = need_dilation ? dilation : 1;
    g->nvox = (int)nvox;
    return MSD_OK;
}

template <typename T>
int make_view(const char *fn, const char *name, int ndim, const void *p, const int64_t *strides, msd::View<T> *v)
{
    if (!p) return fail(MSD_ERR_INVALID, "%s: %s is NULL", fn, name);
    if (!strides) return fail(MSD_ERR_INVALID, "%s: %s_strides is NULL", fn, name);
    for (int i = 0; i < ndim + 2; i++)
        if (strides[i] < 0) return fail(MSD_ERR_INVALID, "%s: %s has a negative stride", fn, name);
    v->p = (T *)p;
    v->sb = strides[0];
    v->sc = strides[1];
    v->sz = ndim == 3 ? strides[2] : 0;
    v->sy = strides[ndim];
    v->sx = strides[ndim + 1];
    return MSD_OK;
}

int check_workspace(const char *fn, const msd::Geom &g, size_t elem, const void *ws, int64_t bytes)
{
    const int64_t need = msd::generic_workspace_elems(g) * (int64_t)elem;
    if (!ws || bytes < need)
        return fail(MSD_ERR_WORKSPACE, "%s: workspace of %lld bytes needed, %lld given", fn, (long long)need,
                    (long long)(ws ? bytes : 0));
    return MSD_OK;
}

#define MSD_TRY(expr)            \
    do {                         \
        int rc_ = (expr);        \
        if (rc_ != MSD_OK) return rc_; \
    } while (0)

template <typename T>
int forward_t(const char *fn, bool relu, const msd::Geom &g, int ndim, const void *input, const int64_t *is,
              const void *kernel, const void *bias, void *output, const int64_t *os, hipStream_t s)
{
    msd::View<const T> x;
    msd::View<T> y;
    MSD_TRY(make_view(fn, "input", ndim, input, is, &x));
    MSD_TRY(make_view(fn, "output", ndim, output, os, &y));
    if (!kernel) return fail(MSD_ERR_INVALID, "%s: kernel is NULL", fn);
    if (!bias) return fail(MSD_ERR_INVALID, "%s: bias is NULL", fn);
    ProfileScope scope(0, s);
    hipError_t e;
    if constexpr (is_f32<T>::value) {
        if (g_kernel_path == 0 && g.Wd > 2 && ndim == 3) {
            // Wider layers in 3D: the specialised kernels take the output channels two at a time
            // (the last group may hold one), where every group qualifies: 128^3, 24 -> 3 channels
            // 171 against 979 us.  (In 2D the shape-generic kernel, which reads the input once for
            // all output channels, is as fast at three and faster at four; likewise the generic
            // weight-gradient kernel in both ranks.)
            const int64_t taps = ndim == 3 ? 27 : 9;
            bool all = true;
            for (int co = 0; co < g.Wd && all; co += 2) {
                msd::Geom g2 = g;
                g2.Wd = std::min(2, g.Wd - co);
                msd::View<float> y2 = y;
                y2.p += (int64_t)co * y.sc;
                all = msd::fast_forward_supported(g2, x, y2);
            }
            if (all) {
                for (int co = 0; co < g.Wd; co += 2) {
                    msd::Geom g2 = g;
                    g2.Wd = std::min(2, g.Wd - co);
                    msd::View<float> y2 = y;
                    y2.p += (int64_t)co * y.sc;
                    e = msd::fast_forward(g2, relu, x, (const float *)kernel + (int64_t)co * g.C * taps,
                                          (const float *)bias + co, y2, s);
                    if (e != hipSuccess) return hip_fail(fn, e);
                }
                return MSD_OK;
            }
        }
        if (g_kernel_path == 0 && msd::fast_forward_supported(g, x, y))
            e = msd::fast_forward(g, relu, x, (const float *)kernel, (const float *)bias, y, s);
        else
            e = msd::generic_forward<T>(g, relu, x, (const T *)kernel, (const T *)bias, y, s);
    } else {
        e = msd::generic_forward<T>(g, relu, x, (const T *)kernel, (const T *)bias, y, s);
    }
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int forward(const char *fn, bool relu, int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
            const int64_t *spatial, int dilation, const void *input, const int64_t *is, const void *kernel,
            const void *bias, void *output, const int64_t *os, void *stream, bool reverse = false)
{
    msd::Geom g;
    MSD_TRY(make_geom(fn, dtype, ndim, batch, c_in, c_out, spatial, dilation, true, &g));
    if (c_in <= 0) return fail(MSD_ERR_INVALID, "%s: c_in must be positive", fn);
    g.reverse = reverse;
    return dtype == MSD_F32
               ? forward_t<float>(fn, relu, g, ndim, input, is, kernel, bias, output, os, (hipStream_t)stream)
               : forward_t<double>(fn, relu, g, ndim, input, is, kernel, bias, output, os, (hipStream_t)stream);
}

template <typename T>
int backward_x_t(const char *fn, bool relu, const msd::Geom &g, int ndim, const void *output, const int64_t *os,
                 const void *grad_output, const int64_t *gs, const void *kernel, void *grad_input,
                 const int64_t *xs, hipStream_t s, int mask_from, const void *act, const int64_t *as, bool *masked)
{
    msd::View<const T> o{nullptr, 0, 0, 0, 0, 0}, gy;
    msd::View<T> gx;
    if (relu) MSD_TRY(make_view(fn, "output", ndim, output, os, &o));
    MSD_TRY(make_view(fn, "grad_output", ndim, grad_output, gs, &gy));
    MSD_TRY(make_view(fn, "grad_input", ndim, grad_input, xs, &gx));
    if (!kernel) return fail(MSD_ERR_INVALID, "%s: kernel is NULL", fn);
    ProfileScope scope(1, s);
    hipError_t e;
    if constexpr (is_f32<T>::value) {
        if (g_kernel_path == 0 && g.Wd > 2) {
            // Wider layers: two output channels at a time, each group adding its share to
            // grad_input (the optional mask on the way out is left to the caller: *masked
            // stays false).  1024^2, 4 -> 48 channels: 138 against 295 us.
            const int64_t taps = ndim == 3 ? 27 : 9;
            auto group = [&](int co, msd::Geom *g2, msd::View<const float> *o2, msd::View<const float> *gy2) {
                *g2 = g;
                g2->Wd = std::min(2, g.Wd - co);
                *o2 = o;
                if (relu) o2->p += (int64_t)co * o.sc;
                *gy2 = gy;
                gy2->p += (int64_t)co * gy.sc;
            };
            bool all = true;
            for (int co = 0; co < g.Wd && all; co += 2) {
                msd::Geom g2;
                msd::View<const float> o2, gy2;
                group(co, &g2, &o2, &gy2);
                all = msd::fast_backward_x_supported(g2, relu, o2, gy2, gx);
            }
            if (all) {
                const msd::PostMask none{g.C, {nullptr, 0, 0, 0, 0, 0}};
                for (int co = 0; co < g.Wd; co += 2) {
                    msd::Geom g2;
                    msd::View<const float> o2, gy2;
                    group(co, &g2, &o2, &gy2);
                    e = msd::fast_backward_x(g2, relu, o2, gy2, (const float *)kernel + (int64_t)co * g.C * taps, gx,
                                             none, s);
                    if (e != hipSuccess) return hip_fail(fn, e);
                }
                return MSD_OK;
            }
        }
        if (g_kernel_path == 0 && msd::fast_backward_x_supported(g, relu, o, gy, gx)) {
            msd::PostMask pm{g.C, {nullptr, 0, 0, 0, 0, 0}};
            if (act && as && as[ndim + 1] == 1) {
                // the activation view must allow the same aligned V-wide loads as grad_input
                msd::View<const float> av;
                MSD_TRY(make_view(fn, "activation", ndim, act, as, &av));
                const bool same_layout = av.sb == gx.sb && av.sc == gx.sc && av.sz == gx.sz && av.sy == gx.sy &&
                                         reinterpret_cast<uintptr_t>(av.p) % 16 == reinterpret_cast<uintptr_t>(gx.p) % 16;
                if (same_layout) {
                    pm = msd::PostMask{mask_from, av};
                    if (masked) *masked = true;
                }
            }
            e = msd::fast_backward_x(g, relu, o, gy, (const float *)kernel, gx, pm, s);
        } else
            e = msd::generic_backward_x<T>(g, relu, o, gy, (const T *)kernel, gx, s);
    } else {
        e = msd::generic_backward_x<T>(g, relu, o, gy, (const T *)kernel, gx, s);
    }
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int backward_x(const char *fn, bool relu, int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
               const int64_t *spatial, int dilation, const void *output, const int64_t *os, const void *grad_output,
               const int64_t *gs, const void *kernel, void *grad_input, const int64_t *xs, void *stream,
               int mask_from = 0, const void *act = nullptr, const int64_t *as = nullptr, bool *masked = nullptr)
{
    // act/as/mask_from: optional ReLU mask applied to grad_input channels >= mask_from on the
    // way out (dense block only); *masked reports whether the kernel that ran did it.
    msd::Geom g;
    MSD_TRY(make_geom(fn, dtype, ndim, batch, c_in, c_out, spatial, dilation, true, &g));
    if (c_in <= 0) return fail(MSD_ERR_INVALID, "%s: c_in must be positive", fn);
    if (masked) *masked = false;
    return dtype == MSD_F32 ? backward_x_t<float>(fn, relu, g, ndim, output, os, grad_output, gs, kernel, grad_input,
                                                  xs, (hipStream_t)stream, mask_from, act, as, masked)
                            : backward_x_t<double>(fn, relu, g, ndim, output, os, grad_output, gs, kernel, grad_input,
                                                   xs, (hipStream_t)stream, mask_from, act, as, masked);
}

template <typename T>
int backward_kb_t(const char *fn, bool relu, const msd::Geom &g, int ndim, const void *output, const int64_t *os,
                  const void *grad_output, const int64_t *gs, const void *input, const int64_t *xs, void *grad_kernel,
                  void *grad_bias, void *ws, int64_t ws_bytes, hipStream_t s)
{
    msd::View<const T> o{nullptr, 0, 0, 0, 0, 0}, gy, x{nullptr, 0, 0, 0, 0, 0};
    if (relu) MSD_TRY(make_view(fn, "output", ndim, output, os, &o));
    MSD_TRY(make_view(fn, "grad_output", ndim, grad_output, gs, &gy));
    if (grad_kernel) MSD_TRY(make_view(fn, "input", ndim, input, xs, &x));
    if (!grad_kernel && !grad_bias) return fail(MSD_ERR_INVALID, "%s: no gradient buffer given", fn);
    MSD_TRY(check_workspace(fn, g, sizeof(T), ws, ws_bytes));
    ProfileScope scope(2, s);
    hipError_t e;
    if constexpr (is_f32<T>::value) {
        if (g_kernel_path == 0 && grad_kernel && msd::fast_backward_kb_supported(g, relu, o, gy, x))
            e = msd::fast_backward_kb(g, relu, o, gy, x, (float *)grad_kernel, (float *)grad_bias, (float *)ws, s);
        else
            e = msd::generic_backward_kb<T>(g, relu, o, gy, x, (T *)grad_kernel, (T *)grad_bias, (T *)ws, s);
    } else {
        e = msd::generic_backward_kb<T>(g, relu, o, gy, x, (T *)grad_kernel, (T *)grad_bias, (T *)ws, s);
    }
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int backward_kb(const char *fn, bool relu, bool need_k, int dtype, int ndim, int64_t batch, int64_t c_in,
                int64_t c_out, const int64_t *spatial, int dilation, const void *output, const int64_t *os,
                const void *grad_output, const int64_t *gs, const void *input, const int64_t *xs, void *grad_kernel,
                void *grad_bias, void *ws, int64_t ws_bytes, void *stream)
{
    msd::Geom g;
    MSD_TRY(make_geom(fn, dtype, ndim, batch, c_in, c_out, spatial, dilation, need_k, &g));
    if (need_k && c_in <= 0) return fail(MSD_ERR_INVALID, "%s: c_in must be positive", fn);
    if (need_k && !grad_kernel) return fail(MSD_ERR_INVALID, "%s: grad_kernel is NULL", fn);
    return dtype == MSD_F32 ? backward_kb_t<float>(fn, relu, g, ndim, output, os, grad_output, gs, input, xs,
                                                   grad_kernel, grad_bias, ws, ws_bytes, (hipStream_t)stream)
                            : backward_kb_t<double>(fn, relu, g, ndim, output, os, grad_output, gs, input, xs,
                                                    grad_kernel, grad_bias, ws, ws_bytes, (hipStream_t)stream);
}

}  // namespace

extern "C" {

const char *msd_last_error(void) { return g_error.c_str(); }

int msd_abi_version(void) { return 1; }

int msd_set_tuning(const char *key, int value)
{
    if (!key) return fail(MSD_ERR_INVALID, "msd_set_tuning: key is NULL");
    for (int i = 0; i < msd::kKnobCount; i++)
        if (std::string(key) == msd::kKnobNames[i]) {
            msd::g_knobs[i] = value;
            return MSD_OK;
        }
    return fail(MSD_ERR_INVALID, "msd_set_tuning: unknown key '%s'", key);
}

int msd_set_kernel_path(int path)
{
    if (path != 0 && path != 1) return fail(MSD_ERR_INVALID, "msd_set_kernel_path: path must be 0 or 1");
    g_kernel_path = path;
    return MSD_OK;
}

int64_t msd_workspace_bytes(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial)
{
    msd::Geom g;
    if (make_geom("msd_workspace_bytes", dtype, ndim, batch, c_in, c_out, spatial, 1, false, &g) != MSD_OK) return -1;
    return msd::generic_workspace_elems(g) * (dtype == MSD_F32 ? 4 : 8);
}

int msd_conv_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                     int dilation, const void *input, const int64_t *input_strides, const void *kernel,
                     const void *bias, void *output, const int64_t *output_strides, void *stream)
{
    return forward("conv_forward", false, dtype, ndim, batch, c_in, c_out, spatial, dilation, input, input_strides,
                   kernel, bias, output, output_strides, stream);
}

int msd_conv_relu_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                          int dilation, const void *input, const int64_t *input_strides, const void *kernel,
                          const void *bias, void *output, const int64_t *output_strides, void *stream)
{
    return forward("conv_relu_forward", true, dtype, ndim, batch, c_in, c_out, spatial, dilation, input,
                   input_strides, kernel, bias, output, output_strides, stream);
}

int msd_conv_backward_x(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                        int dilation, const void *grad_output, const int64_t *grad_output_strides, const void *kernel,
                        void *grad_input, const int64_t *grad_input_strides, void *stream)
{
    return backward_x("conv_backward_x", false, dtype, ndim, batch, c_in, c_out, spatial, dilation, nullptr, nullptr,
                      grad_output, grad_output_strides, kernel, grad_input, grad_input_strides, stream);
}

int msd_conv_relu_backward_x(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                             int dilation, const void *output, const int64_t *output_strides, const void *grad_output,
                             const int64_t *grad_output_strides, const void *kernel, void *grad_input,
                             const int64_t *grad_input_strides, void *stream)
{
    return backward_x("conv_relu_backward_x", true, dtype, ndim, batch, c_in, c_out, spatial, dilation, output,
                      output_strides, grad_output, grad_output_strides, kernel, grad_input, grad_input_strides, stream);
}

int msd_conv_backward_k(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                        int dilation, const void *grad_output, const int64_t *grad_output_strides, const void *input,
                        const int64_t *input_strides, void *grad_kernel, void *workspace, int64_t workspace_bytes,
                        void *stream)
{
    return backward_kb("conv_backward_k", false, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, nullptr,
                       nullptr, grad_output, grad_output_strides, input, input_strides, grad_kernel, nullptr,
                       workspace, workspace_bytes, stream);
}

int msd_conv_relu_backward_k(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                             int dilation, const void *output, const int64_t *output_strides, const void *grad_output,
                             const int64_t *grad_output_strides, const void *input, const int64_t *input_strides,
                             void *grad_kernel, void *workspace, int64_t workspace_bytes, void *stream)
{
    return backward_kb("conv_relu_backward_k", true, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, output,
                       output_strides, grad_output, grad_output_strides, input, input_strides, grad_kernel, nullptr,
                       workspace, workspace_bytes, stream);
}

int msd_conv_backward_bias(int dtype, int ndim, int64_t batch, int64_t c_out, const int64_t *spatial,
                           const void *grad_output, const int64_t *grad_output_strides, void *grad_bias,
                           void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!grad_bias) return fail(MSD_ERR_INVALID, "conv_backward_bias: grad_bias is NULL");
    return backward_kb("conv_backward_bias", false, false, dtype, ndim, batch, 0, c_out, spatial, 1, nullptr, nullptr,
                       grad_output, grad_output_strides, nullptr, nullptr, nullptr, grad_bias, workspace,
                       workspace_bytes, stream);
}

int msd_conv_relu_backward_bias(int dtype, int ndim, int64_t batch, int64_t c_out, const int64_t *spatial,
                                const void *output, const int64_t *output_strides, const void *grad_output,
                                const int64_t *grad_output_strides, void *grad_bias, void *workspace,
                                int64_t workspace_bytes, void *stream)
{
    if (!grad_bias) return fail(MSD_ERR_INVALID, "conv_relu_backward_bias: grad_bias is NULL");
    return backward_kb("conv_relu_backward_bias", true, false, dtype, ndim, batch, 0, c_out, spatial, 1, output,
                       output_strides, grad_output, grad_output_strides, nullptr, nullptr, nullptr, grad_bias,
                       workspace, workspace_bytes, stream);
}

int msd_conv_backward_kb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                         int dilation, const void *grad_output, const int64_t *grad_output_strides, const void *input,
                         const int64_t *input_strides, void *grad_kernel, void *grad_bias, void *workspace,
                         int64_t workspace_bytes, void *stream)
{
    return backward_kb("conv_backward_kb", false, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, nullptr,
                       nullptr, grad_output, grad_output_strides, input, input_strides, grad_kernel, grad_bias,
                       workspace, workspace_bytes, stream);
}

int msd_conv_backward_xkb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                          int dilation, const void *grad_output, const int64_t *grad_output_strides,
                          const void *input, const int64_t *input_strides, const void *kernel, void *grad_input,
                          const int64_t *grad_input_strides, void *grad_kernel, void *grad_bias, void *workspace,
                          int64_t workspace_bytes, void *stream)
{
    const char *fn = "conv_backward_xkb";
    if (!grad_kernel) return fail(MSD_ERR_INVALID, "%s: grad_kernel is NULL", fn);
    if (dtype == MSD_F32 && g_kernel_path == 0 && ndim >= 2 && ndim <= 3) {
        // one pass where the fused kernel covers the case
        msd::Geom g;
        MSD_TRY(make_geom(fn, dtype, ndim, batch, c_in, c_out, spatial, dilation, true, &g));
        if (c_in <= 0) return fail(MSD_ERR_INVALID, "%s: c_in must be positive", fn);
        if (!kernel) return fail(MSD_ERR_INVALID, "%s: kernel is NULL", fn);
        msd::View<const float> gy, x;
        msd::View<float> gx;
        MSD_TRY(make_view(fn, "grad_output", ndim, grad_output, grad_output_strides, &gy));
        MSD_TRY(make_view(fn, "input", ndim, input, input_strides, &x));
        MSD_TRY(make_view(fn, "grad_input", ndim, grad_input, grad_input_strides, &gx));
        if (msd::fast_backward_xkb_supported(g, gy, x, gx)) {
            MSD_TRY(check_workspace(fn, g, sizeof(float), workspace, workspace_bytes));
            const msd::PostMask none{g.C, {nullptr, 0, 0, 0, 0, 0}};
            ProfileScope scope(3, (hipStream_t)stream);
            const hipError_t e =
                msd::fast_backward_xkb(g, gy, x, (const float *)kernel, gx, none, (float *)grad_kernel,
                                       (float *)grad_bias, (float *)workspace, (hipStream_t)stream);
            return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
        }
    }
    MSD_TRY(backward_x(fn, false, dtype, ndim, batch, c_in, c_out, spatial, dilation, nullptr, nullptr, grad_output,
                       grad_output_strides, kernel, grad_input, grad_input_strides, stream));
    return backward_kb(fn, false, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, nullptr, nullptr,
                       grad_output, grad_output_strides, input, input_strides, grad_kernel, grad_bias, workspace,
                       workspace_bytes, stream);
}

int msd_relu_mask_gradient(int dtype, int ndim, int64_t batch, int64_t c_out, const int64_t *spatial,
                           const void *output, const int64_t *output_strides, void *grad_output,
                           const int64_t *grad_output_strides, void *stream)
{
    const char *fn = "relu_mask_gradient";
    msd::Geom g;
    MSD_TRY(make_geom(fn, dtype, ndim, batch, 0, c_out, spatial, 1, false, &g));
    ProfileScope scope(1, (hipStream_t)stream);
    if (dtype == MSD_F32) {
        msd::View<const float> o;
        msd::View<float> gy;
        MSD_TRY(make_view(fn, "output", ndim, output, output_strides, &o));
        MSD_TRY(make_view(fn, "grad_output", ndim, grad_output, grad_output_strides, &gy));
        hipError_t e = msd::generic_relu_mask<float>(g, o, gy, (hipStream_t)stream);
        return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
    }
    msd::View<const double> o;
    msd::View<double> gy;
    MSD_TRY(make_view(fn, "output", ndim, output, output_strides, &o));
    MSD_TRY(make_view(fn, "grad_output", ndim, grad_output, grad_output_strides, &gy));
    hipError_t e = msd::generic_relu_mask<double>(g, o, gy, (hipStream_t)stream);
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int msd_conv_relu_backward_kb(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out, const int64_t *spatial,
                              int dilation, const void *output, const int64_t *output_strides, const void *grad_output,
                              const int64_t *grad_output_strides, const void *input, const int64_t *input_strides,
                              void *grad_kernel, void *grad_bias, void *workspace, int64_t workspace_bytes,
                              void *stream)
{
    return backward_kb("conv_relu_backward_kb", true, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, output,
                       output_strides, grad_output, grad_output_strides, input, input_strides, grad_kernel, grad_bias,
                       workspace, workspace_bytes, stream);
}


// ---------------------------------------------------------------------------
// msd_conv_relu_backward_kb for callers that cannot allocate: the partial sums go through
// a buffer that is part of the library's device image instead of a caller's workspace.
// ---------------------------------------------------------------------------

// One copy per GPU the library runs on, held until the process ends.  In host code this name
// is only a handle for hipGetSymbolAddress: it is not a device address.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[MSD_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];   // device address of `scratch` on device i, once looked up

// Address of the current device's copy of `scratch` (looked up on the first call on each
// device, with that device current).
int static_scratch(const char *fn, void **ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(fn, e);
    if (dev < 0 || dev >= kMaxDevices) return fail(MSD_ERR_INVALID, "%s: device index %d not supported", fn, dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(fn, e);
        if (!p) return fail(MSD_ERR_HIP, "%s: the static scratch buffer has no device address", fn);
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return MSD_OK;
}

}  // namespace

int msd_conv_relu_backward_kb_static(int dtype, int ndim, int64_t batch, int64_t c_in, int64_t c_out,
                                     const int64_t *spatial, int dilation, const void *output,
                                     const int64_t *output_strides, const void *grad_output,
                                     const int64_t *grad_output_strides, const void *input,
                                     const int64_t *input_strides, void *grad_kernel, void *grad_bias, void *stream)
{
    const char *fn = "conv_relu_backward_kb_static";
    // geometry and size first: these rejections touch no device
    msd::Geom g;
    MSD_TRY(make_geom(fn, dtype, ndim, batch, c_in, c_out, spatial, dilation, true, &g));
    if (c_in <= 0) return fail(MSD_ERR_INVALID, "%s: c_in must be positive", fn);
    const int64_t need = msd::generic_workspace_elems(g) * (dtype == MSD_F32 ? 4 : 8);
    if (need > MSD_STATIC_SCRATCH_BYTES)
        return fail(MSD_ERR_WORKSPACE,
                    "%s: this problem needs %lld bytes of scratch, the library's static buffer holds %lld; "
                    "call msd_conv_relu_backward_kb with a workspace instead",
                    fn, (long long)need, (long long)MSD_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    MSD_TRY(static_scratch(fn, &ws));
    // the kernels write every partial sum (and every value of the masked gradient) that the
    // second pass reads, so nothing in the buffer has to start at zero
    return backward_kb(fn, true, true, dtype, ndim, batch, c_in, c_out, spatial, dilation, output, output_strides,
                       grad_output, grad_output_strides, input, input_strides, grad_kernel, grad_bias, ws,
                       MSD_STATIC_SCRATCH_BYTES, stream);
}

// ---------------------------------------------------------------------------
// Dense block: the layer loops of msd_block.py:40-58 (forward) and :89-130
// (backward) as one native call each, so a training step costs two library calls
// per block instead of four Python-level operator calls per layer.
// ---------------------------------------------------------------------------

namespace {

struct BlockArgs {
    int dtype, ndim, depth;
    int64_t batch, c_in, c_total;
    const int64_t *widths, *spatial, *dilations;
    size_t elem;
};

int check_block(const char *fn, int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                const int64_t *spatial, const int64_t *dilations, const void *stack, const int64_t *stack_strides,
                const void *const *weights, BlockArgs *a)
{
    if (dtype != MSD_F32 && dtype != MSD_F64) return fail(MSD_ERR_INVALID, "%s: dtype must be MSD_F32 or MSD_F64", fn);
    if (ndim != 2 && ndim != 3) return fail(MSD_ERR_INVALID, "%s: expected 2 or 3 spatial dimensions, got %d", fn, ndim);
    if (depth <= 0 || c_in <= 0 || batch <= 0) return fail(MSD_ERR_INVALID, "%s: depth, c_in and batch must be positive", fn);
    if (!widths || !spatial || !dilations || !stack || !stack_strides || !weights)
        return fail(MSD_ERR_INVALID, "%s: NULL argument", fn);
    int64_t total = c_in;
    for (int i = 0; i < depth; i++) {
        if (widths[i] <= 0) return fail(MSD_ERR_INVALID, "%s: layer widths must be positive", fn);
        if (!weights[i]) return fail(MSD_ERR_INVALID, "%s: weights[%d] is NULL", fn, i);
        if (dilations[i] <= 0) return fail(MSD_ERR_INVALID, "%s: Dilation must be 1 or greater", fn);
        for (int d = 0; d < ndim; d++)
            if (dilations[i] > spatial[d])
                return fail(MSD_ERR_INVALID, "%s: Dilation cannot be greater than size of image.", fn);
        total += widths[i];
    }
    *a = BlockArgs{dtype, ndim, depth, batch, c_in, total, widths, spatial, dilations, dtype == MSD_F32 ? 4u : 8u};
    return MSD_OK;
}


// One layer of the block backward pass with the fused kernel: grad_input channels
// [0, first) += backward_x, grad_weights/grad_bias += backward_k/bias, the ReLU mask of the
// layer below applied to its channels on the way out.  *done is false (and nothing was
// launched) when the fused kernel does not cover the case.
// Floats of workspace that the partial sums of one fused layer take.
int64_t partial_region_floats(int ndim, int64_t c_in, int64_t width)
{
    return width * (c_in * (ndim == 3 ? 27 : 9) + 1) * (int64_t)msd::kMaxPartialRows;
}

constexpr int64_t kDeferBudgetBytes = (int64_t)1 << 30;   // most workspace spent on pending partial sums

// Largest workspace a single layer of the block asks for, rounded up to 256 bytes: the
// regions of the pending reductions start there.
int64_t block_layer_workspace(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                              const int64_t *spatial)
{
    int64_t total = c_in, need = 0;
    for (int i = 0; i < depth; i++) {
        if (widths[i] <= 0) return -1;
        int64_t n = msd_workspace_bytes(dtype, ndim, batch, total, widths[i], spatial);
        if (n < 0) return -1;
        if (ndim == 3 && i + 1 < depth && widths[i + 1] == 1 && widths[i] == 1) {
            // 3D: the weight gradients of this layer and the one above it in one pass
            const int64_t nup = msd_workspace_bytes(dtype, ndim, batch, total + 1, 2, spatial);
            n = nup > n ? nup : n;
        }
        for (int up = 1; up < msd::kMaxLayerGroup; up++) {
            // this layer and the one or two above it may run as the output channels of one pass
            if (ndim != 2 || i + up >= depth || widths[i + up] != 1 || widths[i] != 1) break;
            const int64_t nup = msd_workspace_bytes(dtype, ndim, batch, total, up + 1, spatial);
            n = nup > n ? nup : n;
        }
        need = n > need ? n : need;
        total += widths[i];
    }
    return (need + 255) / 256 * 256;
}

// The reverse loop's pending column reductions: each fused layer leaves its partial sums in
// a region of its own behind the per-layer workspace, and one launch reduces up to
// kReduceBatch layers (a reduction per layer is a 4 microsecond launch between two large
// kernels).  With no room for regions every layer reduces at once, as the single operators do.
struct DeferredReductions {
    float *base = nullptr;
    int64_t capacity = 0, cursor = 0;             // floats
    msd::ReduceJob jobs[msd::kReduceBatch];
    int n = 0;
    hipStream_t s = nullptr;

    int flush(const char *fn)
    {
        if (n == 0) return MSD_OK;
        ProfileScope scope(3, s, false);
        const hipError_t e = msd::reduce_columns_batch(jobs, n, s);
        n = 0;
        cursor = 0;
        return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
    }
    // the job to hand to the next fused layer, its region set; nullptr when the region cannot fit
    int next(const char *fn, int64_t floats, msd::ReduceJob **job)
    {
        *job = nullptr;
        if (!base || floats > capacity) return MSD_OK;
        if (n == msd::kReduceBatch || cursor + floats > capacity) MSD_TRY(flush(fn));
        jobs[n].part = base + cursor;
        *job = &jobs[n];
        return MSD_OK;
    }
    void taken(int64_t floats)
    {
        n++;
        cursor += floats;
    }
};

int block_layer_fused(const char *fn, const BlockArgs &a, int i, int64_t first, const void *stack,
                      const int64_t *stack_strides, void *grads, const int64_t *grads_strides, const void *gout_i,
                      const void *weights_i, void *gk, void *gb, void *ws, int64_t ws_bytes, hipStream_t s,
                      DeferredReductions *pending, bool *masked, bool *done)
{
    *done = false;
    if (a.dtype != MSD_F32 || g_kernel_path != 0 || !gk || !msd::knob(msd::kKnobBlockFuse, 1)) return MSD_OK;
    msd::Geom g;
    MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, first, a.widths[i], a.spatial, (int)a.dilations[i], true, &g));
    msd::View<const float> gy, x;
    msd::View<float> gx;
    MSD_TRY(make_view(fn, "grad_output", a.ndim, gout_i, grads_strides, &gy));
    MSD_TRY(make_view(fn, "input", a.ndim, stack, stack_strides, &x));
    MSD_TRY(make_view(fn, "grad_input", a.ndim, grads, grads_strides, &gx));
    if (!msd::fast_backward_xkb_supported(g, gy, x, gx)) return MSD_OK;
    MSD_TRY(check_workspace(fn, g, sizeof(float), ws, ws_bytes));
    msd::PostMask pm{g.C, {nullptr, 0, 0, 0, 0, 0}};
    *masked = false;
    if (i > 0) {
        // the activations are read through grad_input's addressing: same strides and alignment
        const bool same_layout = x.sb == gx.sb && x.sc == gx.sc && x.sz == gx.sz && x.sy == gx.sy &&
                                 reinterpret_cast<uintptr_t>(x.p) % 16 == reinterpret_cast<uintptr_t>(gx.p) % 16;
        if (same_layout) {
            pm = msd::PostMask{(int)(first - a.widths[i - 1]), x};
            *masked = true;
        }
    }
    const int64_t region = partial_region_floats(a.ndim, g.C, g.Wd);
    msd::ReduceJob *job = nullptr;
    MSD_TRY(pending->next(fn, region, &job));
    ProfileScope scope(3, s);
    // as in the forward loop: alternate layers walk the channels in opposite directions
    g.reverse = msd::knob(msd::kKnobBlockSnake, 1) && (i & 1);
    const hipError_t e = msd::fast_backward_xkb(g, gy, x, (const float *)weights_i, gx, pm, (float *)gk, (float *)gb,
                                                (float *)ws, s, job);
    if (e != hipSuccess) return hip_fail(fn, e);
    if (job) pending->taken(region);
    *done = true;
    return MSD_OK;
}

// A group of n = 2 or 3 layers of the block backward pass, i down to i - n + 1 (2D, one output
// channel each), in n launches instead of n full passes.  Layer i's inputs are the channels
// [0, first), those of the lowest layer of the group the channels [0, c), c = first - (n - 1);
// channel first - j is layer i - j's output.
//   1. the top j layers of the group on channel first - j alone, for j = 1 .. n - 1: their
//      grad_input contributions complete that channel's gradient (masked with the channel's
//      activation on the way out: it is layer i - j's output gradient from here on), plus the
//      nine weight gradients of that channel per layer;
//   2. all n layers on the channels [0, c) as the output channels of ONE pass of the fused
//      kernel (each with its own dilation and weights): every channel of the input and of
//      grad_input is moved once for the n layers, and their bias gradients are formed there.
// *done is false (and nothing was launched) when the case is not covered.
bool group_candidate(const BlockArgs &a, int i, int n, bool need_input_grad)
{
    if (a.dtype != MSD_F32 || a.ndim != 2 || g_kernel_path != 0 || i - (n - 1) < 0) return false;
    for (int j = 0; j < n; j++)
        if (a.widths[i - j] != 1) return false;
    return (i - (n - 1) > 0 || need_input_grad) && msd::knob(msd::kKnobBlockFuse, 1) &&
           msd::knob(msd::kKnobBlockPair, 1);
}

// Layers to take together from layer i down, most first.  Three where the shared pass is over
// enough channels to gain from it (its tiles cost more to set up than a pair's): 32, or the
// value of "block.triple" (1: wherever possible; 0: never).
int group_sizes(const BlockArgs &a, int i, int64_t first, bool need_input_grad, int (&sizes)[2])
{
    int m = 0;
    const int triple = msd::knob(msd::kKnobBlockTriple, -1);
    const int64_t from_channels = triple < 0 ? 32 : triple;
    if (triple != 0 && group_candidate(a, i, 3, need_input_grad) && first - 2 >= from_channels)
        sizes[m++] = 3;
    if (group_candidate(a, i, 2, need_input_grad)) sizes[m++] = 2;
    return m;
}

int block_group_fused(const char *fn, const BlockArgs &a, int i, int n, int64_t first, const void *stack,
                      const int64_t *stack_strides, void *grads, const int64_t *grads_strides,
                      const void *const *weights, void *const *grad_weights, void *gb_lowest, void *ws,
                      int64_t ws_bytes, hipStream_t s, DeferredReductions *pending, int pass_no, bool *masked,
                      bool *done)
{
    *done = false;
    if (n < 2 || n > msd::kMaxLayerGroup || !gb_lowest) return MSD_OK;
    for (int j = 0; j < n; j++)
        if (!grad_weights[i - j]) return MSD_OK;
    const int lo = i - (n - 1);                   // lowest layer of the group
    const int64_t c = first - (n - 1);            // channels below all layers of the group
    constexpr int K = 9;
    msd::View<const float> x;
    msd::View<float> gx;
    MSD_TRY(make_view(fn, "input", a.ndim, stack, stack_strides, &x));
    MSD_TRY(make_view(fn, "grad_input", a.ndim, grads, grads_strides, &gx));
    // the activations are read through grad_input's addressing: same strides and alignment
    const bool same_layout = x.sb == gx.sb && x.sc == gx.sc && x.sz == gx.sz && x.sy == gx.sy &&
                             reinterpret_cast<uintptr_t>(x.p) % 16 == reinterpret_cast<uintptr_t>(gx.p) % 16;
    if (!same_layout) return MSD_OK;
    // launch j = 1 .. n - 1: the top j layers on channel first - j; launch n: all on [0, c)
    struct Step {
        msd::Geom g;
        msd::View<const float> gy, x;
        msd::View<float> gx;
        msd::LayerGroup group;
        const float *k;
        float *gk;
        bool lean;
    } steps[msd::kMaxLayerGroup];
    for (int j = 1; j <= n; j++) {
        Step &st = steps[j - 1];
        const bool shared = j == n;               // the pass over the channels all layers read
        const int64_t ch = shared ? 0 : first - j, chans = shared ? c : 1;
        const int bottom = i - j + 1;             // output channel 0 of this launch
        int dmax = 0;
        st.group.n = j;
        st.group.lowest_channels = 0;
        st.group.max_workgroups = 0;
        for (int q = 0; q < j; q++) {
            st.group.dil[q] = (int)a.dilations[bottom + q];
            dmax = st.group.dil[q] > dmax ? st.group.dil[q] : dmax;
            if (q > 0) {
                st.group.k_up[q - 1] = (const float *)weights[bottom + q] + ch * K;
                st.group.gk_up[q - 1] = (float *)grad_weights[bottom + q] + ch * K;
            }
        }
        st.k = (const float *)weights[bottom] + ch * K;
        st.gk = (float *)grad_weights[bottom] + ch * K;
        MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, chans, j, a.spatial, dmax, true, &st.g));
        st.x = x;
        st.x.p += ch * x.sc;
        st.gx = gx;
        st.gx.p += ch * gx.sc;
        // the output gradients of the launch's layers: the channels above the highest one it updates
        const int64_t gy_ch = shared ? c : ch + 1;
        st.gy = msd::View<const float>{gx.p + gy_ch * gx.sc, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
        st.lean = !shared && msd::fast_backward_one_channel_supported_2d(st.g, st.gy, st.x, st.gx);
        if (!st.lean && !msd::fast_backward_xkb_supported(st.g, st.gy, st.x, st.gx)) return MSD_OK;
        MSD_TRY(check_workspace(fn, st.g, sizeof(float), ws, ws_bytes));
    }
    for (int j = 1; j <= n; j++) {
        Step &st = steps[j - 1];
        const bool shared = j == n;
        // a single channel is an output of the layer below: masked on the way out; the shared
        // pass completes the outputs of layer lo - 1
        msd::PostMask pm{0, st.x};
        if (shared) {
            pm = msd::PostMask{st.g.C, {nullptr, 0, 0, 0, 0, 0}};
            *masked = false;
            if (lo - 1 >= 0) {
                pm = msd::PostMask{(int)(c - a.widths[lo - 1]), x};
                *masked = true;
            }
            st.g.reverse = msd::knob(msd::kKnobBlockSnake, 1) && !(pass_no & 1);
        }
        const int64_t region = partial_region_floats(a.ndim, st.g.C, j);
        msd::ReduceJob *job = nullptr;
        MSD_TRY(pending->next(fn, region, &job));
        ProfileScope scope(3, s);
        const msd::LayerGroup *grp = j > 1 ? &st.group : nullptr;
        const hipError_t e =
            st.lean ? msd::fast_backward_one_channel_2d(st.g, st.gy, st.x, st.k, st.gx, pm, st.gk, (float *)ws, s, job,
                                                        grp)
                    : msd::fast_backward_xkb_2d(st.g, st.gy, st.x, st.k, st.gx, pm, st.gk,
                                                shared ? (float *)gb_lowest : nullptr, (float *)ws, s, job, grp);
        if (e != hipSuccess) return hip_fail(fn, e);
        if (job) pending->taken(region);
    }
    *done = true;
    return MSD_OK;
}

// ---------------------------------------------------------------------------
// 3D blocks of one-channel layers: the reverse loop as two streams of work.
//
// Only the input gradient makes the reverse loop a chain (layer i's masked output gradient
// is complete once every layer above has added its share to that channel); the weight and
// bias gradients of a layer need nothing but that output gradient and the activations.
// So the chain runs as lean backward_x launches (the gather and a read-modify-write stream
// over grad_input, nothing else in registers), and the weight gradients follow on a second
// stream, two layers per pass over x on the matrix cores (fast_backward_k_pair_3d): x is
// read once per two layers, and the chain's launches and the matrix-core launches fill each
// other's gaps.  The second stream is forked from the caller's with an event per pair and
// joined to it before the call returns, so the caller sees one stream's semantics (also
// while its stream is being captured into a graph, once the stream and events exist).
// ---------------------------------------------------------------------------
struct SideStream {
    hipStream_t s = nullptr;
    std::vector<hipEvent_t> events;               // fork events, used in turn; the last one joins
    size_t next = 0;
};
constexpr int kSideEvents = 32;
constexpr int kSideWorkgroups = 384;          // of the weight-gradient pass while the chain runs beside it
std::mutex g_side_mutex;
SideStream g_side[64];

// The current device's second stream, made on first use (default priority); nullptr when it
// cannot be made (the caller then runs everything on its own stream).
SideStream *side_stream()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> lock(g_side_mutex);
    SideStream &side = g_side[dev];
    if (side.s) return &side;
    hipStream_t s = nullptr;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::vector<hipEvent_t> events;
    for (int i = 0; i < kSideEvents + 1; i++) {
        hipEvent_t e;
        if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            for (hipEvent_t made : events) (void)hipEventDestroy(made);
            (void)hipStreamDestroy(s);
            return nullptr;
        }
        events.push_back(e);
    }
    side.s = s;
    side.events = events;
    return &side;
}

// *done is false (and nothing was launched) when the block is not one this path takes.
int block_backward_split3d(const char *fn, const BlockArgs &a, int64_t c_in, const void *stack,
                           const int64_t *stack_strides, void *grads, const int64_t *grads_strides,
                           const void *const *weights, void *const *grad_weights, void *grad_bias, bool need_input_grad,
                           void *workspace, int64_t workspace_bytes, hipStream_t main, DeferredReductions *pending,
                           bool *done)
{
    *done = false;
    // By default wherever the kernels take the shapes: the two streams gain what the launches'
    // ramps and tails leave idle (about 15 to 30 microseconds per launch) and the chain moves half
    // the bytes of grad_input (128^3, depth 50: 6.8 against 8.2 ms for the backward pass; 256^3,
    // depth 30: 35.0 against 35.9 ms per step; 160 x 160 x 256, depth 50: 30.7 against 34.0 ms).
    const int mode = msd::knob(msd::kKnobBlockSplit3d, 1);
    if (mode == 0 || a.dtype != MSD_F32 || a.ndim != 3 || g_kernel_path != 0 || !grad_bias || a.depth < 2 ||
        !msd::knob(msd::kKnobBlockFuse, 1))
        return MSD_OK;
    for (int i = 0; i < a.depth; i++)
        if (a.widths[i] != 1 || !grad_weights[i]) return MSD_OK;
    msd::View<const float> x;
    msd::View<float> gx;
    MSD_TRY(make_view(fn, "input", a.ndim, stack, stack_strides, &x));
    MSD_TRY(make_view(fn, "grad_input", a.ndim, grads, grads_strides, &gx));
    const bool same_layout = x.sb == gx.sb && x.sc == gx.sc && x.sz == gx.sz && x.sy == gx.sy &&
                             reinterpret_cast<uintptr_t>(x.p) % 16 == reinterpret_cast<uintptr_t>(gx.p) % 16;
    if (!same_layout) return MSD_OK;
    // every launch of the plan must be one the specialised kernels take
    struct Pair {
        msd::Geom g;
        msd::LayerGroup group;
        msd::View<const float> gy;
    };
    // The chain takes the same pairs where it can: the upper layer first finishes the one channel
    // the lower layer wrote (a launch over that channel alone), then one read-modify-write pass
    // over the channels below adds both layers' shares (grad_input is read and written once per
    // two layers).  (128^3, depth 50: the chain's launches take 3.2 instead of 4.7 ms.)
    struct Step {
        msd::Geom g;                              // the upper layer over the lower one's channel / the pair's pass
        msd::LayerGroup group;
        msd::View<float> gx;
        const float *k;
        msd::PostMask pm;
    };
    std::vector<Pair> pairs(a.depth);             // pairs[l]: layers (l + 1, l), l the lower one
    std::vector<Step> steps(a.depth);             // [upper]: its one channel; [lower]: the pair's pass
    std::vector<msd::Geom> chain(a.depth);
    bool chain_pairs = msd::knob(msd::kKnobBlockChainPair, 1) != 0 && x.sx == 1;
    const int64_t taps = 27;
    for (int i = a.depth - 1; i >= 0; i--) {
        const int64_t first = c_in + i;           // channels layer i reads; its output is channel `first`
        MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, first, 1, a.spatial, (int)a.dilations[i], true, &chain[i]));
        const msd::View<const float> gy{gx.p + first * gx.sc, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
        if ((i > 0 || need_input_grad) && !msd::fast_backward_x_supported(chain[i], false, gy, gy, gx)) return MSD_OK;
        const bool lower = (a.depth - 1 - i) % 2 == 1;
        if (!lower && i > 0) {
            // layer i over channel first - 1 alone, masked by the activation that channel holds
            Step &st = steps[i];
            MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, 1, 1, a.spatial, (int)a.dilations[i], true, &st.g));
            st.gx = msd::View<float>{gx.p + (first - 1) * gx.sc, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
            st.k = (const float *)weights[i] + (first - 1) * taps;
            st.pm = msd::PostMask{0, {x.p + (first - 1) * x.sc, x.sb, x.sc, x.sz, x.sy, x.sx}};
            chain_pairs = chain_pairs && msd::fast_backward_x_supported(st.g, false, gy, gy, st.gx);
        }
        if (lower) {
            Step &st = steps[i];
            const int du = (int)a.dilations[i + 1], dl = (int)a.dilations[i];
            MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, first, 2, a.spatial, dl, true, &st.g));
            st.group.n = 2;
            st.group.dil[0] = dl;
            st.group.dil[1] = du;
            st.group.dil[2] = 0;
            st.group.k_up[0] = (const float *)weights[i + 1];
            st.group.k_up[1] = nullptr;
            st.group.gk_up[0] = st.group.gk_up[1] = nullptr;
            st.group.lowest_channels = 0;
            st.group.max_workgroups = 0;
            st.gx = gx;
            st.k = (const float *)weights[i];
            st.pm = i > 0 ? msd::PostMask{(int)(first - 1), x} : msd::PostMask{(int)first, {nullptr, 0, 0, 0, 0, 0}};
            if (i > 0 || need_input_grad)
                chain_pairs = chain_pairs && msd::fast_backward_x_pair_supported_3d(st.g, gy, gx);
        }
        if (lower) {
            Pair &p = pairs[i];
            const int du = (int)a.dilations[i + 1], dl = (int)a.dilations[i];
            MSD_TRY(make_geom(fn, a.dtype, a.ndim, a.batch, first + 1, 2, a.spatial, du > dl ? du : dl, true, &p.g));
            p.group.n = 2;
            p.group.dil[0] = dl;
            p.group.dil[1] = du;
            p.group.dil[2] = 0;
            p.group.k_up[0] = p.group.k_up[1] = nullptr;
            p.group.gk_up[0] = (float *)grad_weights[i + 1];
            p.group.gk_up[1] = nullptr;
            p.group.lowest_channels = (int)first;
            p.group.max_workgroups = 0;
            p.gy = gy;                            // channels first (layer i) and first + 1 (layer i + 1)
            if (!msd::fast_backward_k_pair_supported_3d(p.g, p.gy, x)) return MSD_OK;
            MSD_TRY(check_workspace(fn, p.g, sizeof(float), workspace, workspace_bytes));
        }
    }
    // a profiled run keeps to one stream: its per-class event pairs time one stream's work
    SideStream *side = (mode == 1 && !g_profile.on) ? side_stream() : nullptr;
    const hipStream_t ks = side ? side->s : main;
    pending->s = ks;
    auto fork = [&]() -> int {                    // what follows on the second stream waits for the chain so far
        if (!side) return MSD_OK;
        hipEvent_t e;
        {
            std::lock_guard<std::mutex> lock(g_side_mutex);   // (calls from several host threads take turns)
            e = side->events[side->next];
            side->next = (side->next + 1) % kSideEvents;
        }
        hipError_t err = hipEventRecord(e, main);
        if (err == hipSuccess) err = hipStreamWaitEvent(side->s, e, 0);
        return err == hipSuccess ? MSD_OK : hip_fail(fn, err);
    };
    bool masked = false;
    for (int i = a.depth - 1; i >= 0; i--) {
        const int64_t first = c_in + i;
        const char *out_i = (const char *)stack + first * stack_strides[1] * a.elem;
        char *gout_i = (char *)grads + first * grads_strides[1] * a.elem;
        if (!masked)
            MSD_TRY(msd_relu_mask_gradient(a.dtype, a.ndim, a.batch, 1, a.spatial, out_i, stack_strides, gout_i,
                                           grads_strides, main));
        masked = false;
        // the output gradients of layer i (and of layer i + 1) are final here
        const bool lower = (a.depth - 1 - i) % 2 == 1;
        if (lower) {
            Pair &p = pairs[i];
            MSD_TRY(fork());
            const int64_t region = partial_region_floats(a.ndim, p.g.C, 2);
            msd::ReduceJob *job = nullptr;
            MSD_TRY(pending->next(fn, region, &job));
            ProfileScope scope(2, ks);
            p.g.reverse = msd::knob(msd::kKnobBlockSnake, 1) && (i & 2);
            // beside the chain, three quarters of the workgroups that would be resident alone:
            // the chain's workgroups find room on every compute unit (128^3, depth 50: 10.0
            // against 10.2 ms per step; 256^3: 33.9 against 34.9; alone on the chip the full
            // number is faster, 10.8 against 11.8 ms)
            p.group.max_workgroups = side ? kSideWorkgroups : 0;
            const hipError_t e = msd::fast_backward_k_pair_3d(p.g, p.gy, x, (float *)grad_weights[i],
                                                              (float *)grad_bias + i, (float *)workspace, ks, job,
                                                              &p.group);
            if (e != hipSuccess) return hip_fail(fn, e);
            if (job) pending->taken(region);
        } else if (i == 0) {
            // an odd layer is left at the bottom: the single-layer operator
            MSD_TRY(fork());
            MSD_TRY(backward_kb("conv_backward_kb", false, true, a.dtype, a.ndim, a.batch, first, 1, a.spatial,
                                (int)a.dilations[i], nullptr, nullptr, gout_i, grads_strides, stack, stack_strides,
                                grad_weights[i], (char *)grad_bias + i * a.elem, workspace, workspace_bytes, ks));
        }
        const msd::View<const float> gy{gx.p + first * gx.sc, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
        if (chain_pairs && !lower && i > 0) {
            const Step &st = steps[i];
            ProfileScope scope(1, main);
            const hipError_t e = msd::fast_backward_x_3d(st.g, false, gy, gy, st.k, st.gx, st.pm, main);
            if (e != hipSuccess) return hip_fail(fn, e);
            masked = true;
        } else if (chain_pairs && lower) {
            if (i > 0 || need_input_grad) {
                const Step &st = steps[i];
                ProfileScope scope(1, main);
                const hipError_t e = msd::fast_backward_x_pair_3d(st.g, gy, st.k, st.gx, st.pm, main, &st.group);
                if (e != hipSuccess) return hip_fail(fn, e);
                masked = i > 0;
            }
        } else if (i > 0 || need_input_grad) {
            MSD_TRY(backward_x("conv_backward_x", false, a.dtype, a.ndim, a.batch, first, 1, a.spatial,
                               (int)a.dilations[i], nullptr, nullptr, gout_i, grads_strides, weights[i], grads,
                               grads_strides, main, i > 0 ? (int)(first - 1) : (int)first, i > 0 ? stack : nullptr,
                               stack_strides, &masked));
        }
    }
    MSD_TRY(pending->flush(fn));
    if (side) {
        hipEvent_t join = side->events[kSideEvents];
        hipError_t err = hipEventRecord(join, side->s);
        if (err == hipSuccess) err = hipStreamWaitEvent(main, join, 0);
        if (err != hipSuccess) return hip_fail(fn, err);
    }
    *done = true;
    return MSD_OK;
}

}  // namespace

int64_t msd_block_workspace_bytes(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                                  const int64_t *spatial)
{
    if (!widths || depth <= 0) return -1;
    const int64_t need = block_layer_workspace(dtype, ndim, batch, c_in, depth, widths, spatial);
    if (need < 0) return -1;
    // behind it: regions for the partial sums of the layers the fused kernel can take, so that
    // their reductions can wait for one another
    int64_t regions = 0, total = c_in;
    for (int i = 0; i < depth; i++) {
        if (dtype == MSD_F32 && widths[i] <= 2)   // (+ the extra columns of a layer pair's first step)
            regions += (partial_region_floats(ndim, total, widths[i]) + 16 * (int64_t)msd::kMaxPartialRows) *
                       (int64_t)sizeof(float);
        total += widths[i];
    }
    return need + (regions < kDeferBudgetBytes ? regions : kDeferBudgetBytes);
}

int msd_block_forward(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                      const int64_t *spatial, const int64_t *dilations, void *stack, const int64_t *stack_strides,
                      const void *const *weights, const void *bias, void *stream)
{
    const char *fn = "block_forward";
    BlockArgs a;
    MSD_TRY(check_block(fn, dtype, ndim, batch, c_in, depth, widths, spatial, dilations, stack, stack_strides,
                        weights, &a));
    if (!bias) return fail(MSD_ERR_INVALID, "%s: bias is NULL", fn);
    ProfileBatch profile_runs((hipStream_t)stream);
    int64_t first = c_in, b0 = 0;
    for (int i = 0; i < depth; i++) {
        char *out = (char *)stack + first * stack_strides[1] * a.elem;
        // Every second layer walks its input channels from the last to the first: what the
        // layer before touched last is then read first, while it is still in the caches
        // (a few per cent on stacks larger than the 256 MB memory-side cache).
        const bool reverse = msd::knob(msd::kKnobBlockSnake, 1) && (i & 1);
        MSD_TRY(forward("conv_relu_forward", true, dtype, ndim, batch, first, widths[i], spatial, (int)dilations[i],
                        stack, stack_strides, weights[i], (const char *)bias + b0 * a.elem, out, stack_strides,
                        stream, reverse));
        first += widths[i];
        b0 += widths[i];
    }
    return MSD_OK;
}

int msd_block_backward(int dtype, int ndim, int64_t batch, int64_t c_in, int depth, const int64_t *widths,
                       const int64_t *spatial, const int64_t *dilations, const void *stack,
                       const int64_t *stack_strides, void *grads, const int64_t *grads_strides,
                       const void *const *weights, void *const *grad_weights, void *grad_bias, int need_input_grad,
                       void *workspace, int64_t workspace_bytes, void *stream)
{
    const char *fn = "block_backward";
    BlockArgs a;
    MSD_TRY(check_block(fn, dtype, ndim, batch, c_in, depth, widths, spatial, dilations, stack, stack_strides,
                        weights, &a));
    if (!grads || !grads_strides || !grad_weights) return fail(MSD_ERR_INVALID, "%s: NULL argument", fn);
    int64_t last = a.c_total, b1 = a.c_total - c_in;
    ProfileBatch profile_runs((hipStream_t)stream);
    DeferredReductions pending;
    pending.s = (hipStream_t)stream;
    const int64_t layer_ws = block_layer_workspace(dtype, ndim, batch, c_in, depth, widths, spatial);
    if (workspace && layer_ws >= 0 && workspace_bytes > layer_ws && msd::knob(msd::kKnobBlockDefer, 1)) {
        pending.base = (float *)((char *)workspace + layer_ws);
        pending.capacity = (workspace_bytes - layer_ws) / (int64_t)sizeof(float);
    }
    {
        bool done = false;
        MSD_TRY(block_backward_split3d(fn, a, c_in, stack, stack_strides, grads, grads_strides, weights, grad_weights,
                                       grad_bias, need_input_grad != 0, workspace, workspace_bytes, (hipStream_t)stream,
                                       &pending, &done));
        if (done) return MSD_OK;
        pending.s = (hipStream_t)stream;
    }
    bool masked = false;   // the mask of the current layer was already applied by the previous backward_x
    int groups_done = 0;
    for (int i = depth - 1; i >= 0; i--) {
        const int64_t w = widths[i], first = last - w, b0 = b1 - w;
        const char *out_i = (const char *)stack + first * stack_strides[1] * a.elem;
        char *gout_i = (char *)grads + first * grads_strides[1] * a.elem;
        // The layer's slice of the private gradient stack is not read again after this
        // iteration: its ReLU mask is applied once, in place, and the plain operators do
        // the rest.  Where the specialised backward_x runs, the mask of layer i-1 rides
        // on layer i's update of those channels (their last one); otherwise, and for
        // the top layer, a separate pass applies it.
        if (!masked)
            MSD_TRY(msd_relu_mask_gradient(dtype, ndim, batch, w, spatial, out_i, stack_strides, gout_i,
                                           grads_strides, stream));
        masked = false;
        void *gb = grad_bias ? (char *)grad_bias + b0 * a.elem : nullptr;
        {
            // this layer and the one or two below it in launches that move every shared channel once
            int sizes[2];
            const int tries = group_sizes(a, i, first, need_input_grad != 0, sizes);
            bool done = false;
            int n = 0;
            for (int t = 0; t < tries && !done; t++) {
                n = sizes[t];
                MSD_TRY(block_group_fused(fn, a, i, n, first, stack, stack_strides, grads, grads_strides, weights,
                                          grad_weights, grad_bias ? (char *)grad_bias + (b0 - (n - 1)) * a.elem : nullptr,
                                          workspace, workspace_bytes, (hipStream_t)stream, &pending, groups_done,
                                          &masked, &done));
            }
            if (done) {
                groups_done++;
                last = first - (n - 1);
                b1 = b0 - (n - 1);
                i -= n - 1;
                continue;
            }
        }
        if (i > 0 || need_input_grad) {
            // one pass for the input, weight and bias gradients where the fused kernel applies
            bool done = false;
            MSD_TRY(block_layer_fused(fn, a, i, first, stack, stack_strides, grads, grads_strides, gout_i, weights[i],
                                      grad_weights[i], gb, workspace, workspace_bytes, (hipStream_t)stream, &pending,
                                      &masked, &done));
            if (done) {
                last = first;
                b1 = b0;
                continue;
            }
        }
        if (grad_weights[i])
            MSD_TRY(backward_kb("conv_backward_kb", false, true, dtype, ndim, batch, first, w, spatial,
                                (int)dilations[i], nullptr, nullptr, gout_i, grads_strides, stack, stack_strides,
                                grad_weights[i], gb, workspace, workspace_bytes, stream));
        else if (gb)
            MSD_TRY(backward_kb("conv_backward_bias", false, false, dtype, ndim, batch, 0, w, spatial, 1, nullptr,
                                nullptr, gout_i, grads_strides, nullptr, nullptr, nullptr, gb, workspace,
                                workspace_bytes, stream));
        if (i > 0 || need_input_grad)
            MSD_TRY(backward_x("conv_backward_x", false, dtype, ndim, batch, first, w, spatial, (int)dilations[i],
                               nullptr, nullptr, gout_i, grads_strides, weights[i], grads, grads_strides, stream,
                               i > 0 ? (int)(first - widths[i - 1]) : (int)first, i > 0 ? stack : nullptr,
                               stack_strides, &masked));
        last = first;
        b1 = b0;
    }
    return pending.flush(fn);
}

// ---------------------------------------------------------------------------
// Final 1x1 layer (msd_module.py:60-88: Conv1d over the flattened voxels).
// ---------------------------------------------------------------------------

namespace {

int check_final(const char *fn, int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox)
{
    if (dtype != MSD_F32 && dtype != MSD_F64) return fail(MSD_ERR_INVALID, "%s: dtype must be MSD_F32 or MSD_F64", fn);
    if (batch <= 0 || c_in <= 0 || c_out <= 0 || nvox <= 0)
        return fail(MSD_ERR_INVALID, "%s: batch, channel counts and voxel count must be positive", fn);
    if (batch > 65535 || c_in > INT32_MAX || c_out > INT32_MAX)
        return fail(MSD_ERR_INVALID, "%s: batch or channel count too large", fn);
    return MSD_OK;
}

}  // namespace

int64_t msd_final_workspace_bytes(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox)
{
    if (check_final("msd_final_workspace_bytes", dtype, batch, c_in, c_out, nvox) != MSD_OK) return -1;
    return msd::final_workspace_elems(batch, c_in, c_out, nvox) * (dtype == MSD_F32 ? 4 : 8);
}

int msd_final_forward(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox, const void *input,
                      int64_t input_batch_stride, int64_t input_channel_stride, const void *weight, const void *bias,
                      void *output, int64_t output_batch_stride, int64_t output_channel_stride, void *stream)
{
    const char *fn = "final_forward";
    MSD_TRY(check_final(fn, dtype, batch, c_in, c_out, nvox));
    if (!input || !weight || !output) return fail(MSD_ERR_INVALID, "%s: NULL argument", fn);
    if (input_batch_stride < 0 || input_channel_stride < 0 || output_batch_stride < 0 || output_channel_stride < 0)
        return fail(MSD_ERR_INVALID, "%s: negative stride", fn);
    const hipError_t e =
        dtype == MSD_F32
            ? msd::final_forward<float>(batch, (int)c_in, (int)c_out, nvox, (const float *)input, input_batch_stride,
                                        input_channel_stride, (const float *)weight, (const float *)bias,
                                        (float *)output, output_batch_stride, output_channel_stride,
                                        (hipStream_t)stream)
            : msd::final_forward<double>(batch, (int)c_in, (int)c_out, nvox, (const double *)input,
                                         input_batch_stride, input_channel_stride, (const double *)weight,
                                         (const double *)bias, (double *)output, output_batch_stride,
                                         output_channel_stride, (hipStream_t)stream);
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int msd_final_backward(int dtype, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox, const void *input,
                       int64_t input_batch_stride, int64_t input_channel_stride, const void *grad_output,
                       int64_t grad_output_batch_stride, int64_t grad_output_channel_stride, const void *weight,
                       void *grad_input, int64_t grad_input_batch_stride, int64_t grad_input_channel_stride,
                       void *grad_weight, void *grad_bias, void *workspace, int64_t workspace_bytes, void *stream)
{
    const char *fn = "final_backward";
    MSD_TRY(check_final(fn, dtype, batch, c_in, c_out, nvox));
    if (!weight || !grad_output) return fail(MSD_ERR_INVALID, "%s: NULL argument", fn);
    if (!input && (grad_weight || grad_bias))
        return fail(MSD_ERR_INVALID, "%s: input is NULL (it may only be omitted when grad_input is the only gradient)", fn);
    if (input_batch_stride < 0 || input_channel_stride < 0 || grad_output_batch_stride < 0 ||
        grad_output_channel_stride < 0 || grad_input_batch_stride < 0 || grad_input_channel_stride < 0)
        return fail(MSD_ERR_INVALID, "%s: negative stride", fn);
    // the workspace holds the partial sums of the weight and bias gradients: not needed for grad_input alone
    const int64_t need = grad_weight || grad_bias ? msd_final_workspace_bytes(dtype, batch, c_in, c_out, nvox) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(MSD_ERR_WORKSPACE, "%s: workspace of %lld bytes needed, %lld given", fn, (long long)need,
                    (long long)(workspace ? workspace_bytes : 0));
    const hipError_t e =
        dtype == MSD_F32
            ? msd::final_backward<float>(batch, (int)c_in, (int)c_out, nvox, (const float *)input, input_batch_stride,
                                         input_channel_stride, (const float *)grad_output, grad_output_batch_stride,
                                         grad_output_channel_stride, (const float *)weight, (float *)grad_input,
                                         grad_input_batch_stride, grad_input_channel_stride, (float *)grad_weight,
                                         (float *)grad_bias, (float *)workspace, (hipStream_t)stream)
            : msd::final_backward<double>(batch, (int)c_in, (int)c_out, nvox, (const double *)input,
                                          input_batch_stride, input_channel_stride, (const double *)grad_output,
                                          grad_output_batch_stride, grad_output_channel_stride,
                                          (const double *)weight, (double *)grad_input, grad_input_batch_stride,
                                          grad_input_channel_stride, (double *)grad_weight, (double *)grad_bias,
                                          (double *)workspace, (hipStream_t)stream);
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int msd_final_forward_loss(int dtype, int loss_kind, int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox,
                           const void *input, int64_t input_batch_stride, int64_t input_channel_stride,
                           const void *weight, const void *bias, const void *target, int64_t target_batch_stride,
                           int64_t target_channel_stride, void *output, int64_t output_batch_stride,
                           int64_t output_channel_stride, void *grad_output, int64_t grad_output_batch_stride,
                           int64_t grad_output_channel_stride, void *grad_weight, void *grad_bias, void *loss,
                           void *workspace, int64_t workspace_bytes, void *stream)
{
    const char *fn = "final_forward_loss";
    MSD_TRY(check_final(fn, dtype, batch, c_in, c_out, nvox));
    if (loss_kind < MSD_LOSS_MSE || loss_kind > MSD_LOSS_NLL)
        return fail(MSD_ERR_INVALID, "%s: loss_kind must be MSD_LOSS_MSE, MSD_LOSS_L1 or MSD_LOSS_NLL", fn);
    if (c_out > 8) return fail(MSD_ERR_INVALID, "%s: at most 8 output channels", fn);
    if (!input || !weight || !target || !output || !grad_output || !loss)
        return fail(MSD_ERR_INVALID, "%s: NULL argument", fn);
    if (input_batch_stride < 0 || input_channel_stride < 0 || target_batch_stride < 0 || target_channel_stride < 0 ||
        output_batch_stride < 0 || output_channel_stride < 0 || grad_output_batch_stride < 0 ||
        grad_output_channel_stride < 0)
        return fail(MSD_ERR_INVALID, "%s: negative stride", fn);
    const int64_t need = msd_final_workspace_bytes(dtype, batch, c_in, c_out, nvox);
    if (!workspace || workspace_bytes < need)
        return fail(MSD_ERR_WORKSPACE, "%s: workspace of %lld bytes needed, %lld given", fn, (long long)need,
                    (long long)(workspace ? workspace_bytes : 0));
    const hipError_t e =
        dtype == MSD_F32
            ? msd::final_forward_loss<float>(loss_kind, batch, (int)c_in, (int)c_out, nvox, (const float *)input,
                                             input_batch_stride, input_channel_stride, (const float *)weight,
                                             (const float *)bias, target, target_batch_stride, target_channel_stride,
                                             (float *)output, output_batch_stride, output_channel_stride,
                                             (float *)grad_output, grad_output_batch_stride,
                                             grad_output_channel_stride, (float *)grad_weight, (float *)grad_bias,
                                             (float *)loss, (float *)workspace, (hipStream_t)stream)
            : msd::final_forward_loss<double>(loss_kind, batch, (int)c_in, (int)c_out, nvox, (const double *)input,
                                              input_batch_stride, input_channel_stride, (const double *)weight,
                                              (const double *)bias, target, target_batch_stride,
                                              target_channel_stride, (double *)output, output_batch_stride,
                                              output_channel_stride, (double *)grad_output, grad_output_batch_stride,
                                              grad_output_channel_stride, (double *)grad_weight, (double *)grad_bias,
                                              (double *)loss, (double *)workspace, (hipStream_t)stream);
    return e == hipSuccess ? MSD_OK : hip_fail(fn, e);
}

int msd_profile_enable(int on)
{
    g_profile.on = on != 0;
    g_profile.batching = false;
    g_profile.open_cls = -1;
    g_profile.used = 0;
    for (auto &v : g_profile.spans) v.clear();
    return MSD_OK;
}

int msd_profile_read(double *ms, int64_t *calls)
{
    if (!ms || !calls) return fail(MSD_ERR_INVALID, "msd_profile_read: NULL argument");
    for (int c = 0; c < kProfileClasses; c++) {
        double total = 0;
        int64_t ncalls = 0;
        for (const auto &sp : g_profile.spans[c]) {
            hipError_t e = hipEventSynchronize(g_profile.pool[sp.stop]);
            float t = 0;
            if (e == hipSuccess) e = hipEventElapsedTime(&t, g_profile.pool[sp.start], g_profile.pool[sp.stop]);
            if (e != hipSuccess) return hip_fail("msd_profile_read", e);
            total += t;
            ncalls += sp.calls;
        }
        ms[c] = total;
        calls[c] = ncalls;
    }
    return MSD_OK;
}

}  // extern "C"
