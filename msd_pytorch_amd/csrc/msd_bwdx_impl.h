// backward_x for fp32 with unit x-stride and one or two output channels:
//     grad_input[ci][u] += sum_co sum_t k[co][ci][t] * A[co][t](u)
// Each lane owns V consecutive voxels of a row.  The adjoint-form gather
// A[co][t] of the masked output gradient (msd_adjoint.h) is done once and kept
// in registers; the channel loop is then a pure stream over grad_input: one
// vector load, K*V*WOUT fused multiply-adds with wave-uniform weights (scalar
// loads), one vector store.  U channels are in flight per iteration so their
// loads overlap.  Algorithmic traffic: (2C + 2w) * N * 4 bytes.
#pragma once
#include "msd_kernels.h"

#include <algorithm>
#include "msd_rows.h"

namespace msd {

namespace bwdx {

template <int NDIM, bool RELU, int WOUT, int V, int U>
__device__ __forceinline__ void bwdx_rows_body(const Geom &g, const RowTeams &rt, int cch, int remap,
                                               const View<const float> &out, const View<const float> &gy,
                                               const float *__restrict__ k, const View<float> &gx, const PostMask &pm)
{
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K, NPQ = RowTaps<NDIM>::NPQ;
    const int team = threadIdx.x / rt.lpr, lane = threadIdx.x % rt.lpr;
    const int lb = block_for_xcd(blockIdx.x, gridDim.x, remap);
    if (lb * rt.rpw >= rt.nrows) return;   // padding block (whole workgroup)
    const int row = lb * rt.rpw + team;
    const int x0 = lane * V;
    const bool act = row < rt.nrows && x0 < g.W;
    const int rr = min(row, rt.nrows - 1);
    const int y = rr % g.H, z = rr / g.H;
    const int b = blockIdx.y;
    const int c0 = blockIdx.z * cch;
    const int c1 = min(c0 + cch, g.C);

    // adjoint gather, kept in registers for the whole channel loop
    float A[WOUT][K][V];
    {
        float *S = lds + (size_t)team * WOUT * NPQ * V * rt.lpr;
        float own[WOUT][NPQ][V];
        stage_source_rows<NDIM, RELU, WOUT, V>(g, rt, out, gy, b, z, y, lane, act, S, own);
#pragma unroll
        for (int i = 0; i < V; i++) {
            const SideTaps<V> side(x0 + i, g.W, g.dil, rt.lpr);
#pragma unroll
            for (int co = 0; co < WOUT; co++)
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    side.read(S + (size_t)(co * NPQ + pq) * V * rt.lpr, A[co][pq * 3 + 0][i], A[co][pq * 3 + 2][i]);
                    A[co][pq * 3 + 1][i] = own[co][pq][i];
                }
        }
    }
    if (!act) return;

    float *gp = gx.p + (int64_t)b * gx.sb + (int64_t)z * gx.sz + (int64_t)y * gx.sy + x0;
    for (int ci = c0; ci < c1; ci += U) {
        float cur[U][V];
        int cu[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            cu[u] = min(ci + u, c1 - 1);
            load_vec<V>(gp + (int64_t)cu[u] * gx.sc, cur[u]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float s[V];
#pragma unroll
            for (int i = 0; i < V; i++) s[i] = 0.f;
#pragma unroll
            for (int co = 0; co < WOUT; co++) {
                const float *kc = k + ((int64_t)co * g.C + cu[u]) * K;
#pragma unroll
                for (int t = 0; t < K; t++) {
                    const float kv = kc[t];
#pragma unroll
                    for (int i = 0; i < V; i++) s[i] += kv * A[co][t][i];
                }
            }
#pragma unroll
            for (int i = 0; i < V; i++) cur[u][i] += s[i];
            // channels from pm.from on are outputs of the layer below: their gradient is
            // complete with this update, so its ReLU mask is applied on the way out
            if (cu[u] >= pm.from) {
                float a[V];
                load_vec<V>(pm.act.p + (int64_t)b * pm.act.sb + (int64_t)cu[u] * pm.act.sc + (int64_t)z * pm.act.sz +
                                (int64_t)y * pm.act.sy + x0,
                            a);
#pragma unroll
                for (int i = 0; i < V; i++) cur[u][i] = 0.f < a[i] ? cur[u][i] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
            if (ci + u < c1) store_vec<V>(gp + (int64_t)cu[u] * gx.sc, cur[u]);
    }
}

constexpr size_t kMaxLds = 64 * 1024;

template <int NDIM, bool RELU, int WOUT, int V, int U, int MAXT>
__global__ __launch_bounds__(MAXT) void bwdx_rows(Geom g, RowTeams rt, int cch, int remap, View<const float> out,
                                                  View<const float> gy, const float *__restrict__ k, View<float> gx,
                                                  PostMask pm)
{
    bwdx_rows_body<NDIM, RELU, WOUT, V, U>(g, rt, cch, remap, out, gy, k, gx, pm);
}

template <int NDIM, bool RELU, int WOUT, int V, int U>
hipError_t launch(const Geom &g, const View<const float> &out, const View<const float> &gy, const float *k,
                  const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    RowTeams rt;
    make_row_teams(g, V, &rt);
    const int nb = (rt.nrows + rt.rpw - 1) / rt.rpw;
    const size_t lds = staged_floats<NDIM>(rt, WOUT) * rt.rpw * sizeof(float);
    // split the channels over the grid only as far as needed to fill the chip:
    // every chunk repeats the gather
    const int wg_per_kblock = (rt.lpr * rt.rpw + 255) / 256;
    int chunks = knob(kKnobBwdxMinBlocks, 1024) / (nb * g.B * wg_per_kblock);
    chunks = max(1, min(chunks, g.C / 8));
    const int cch = (g.C + chunks - 1) / chunks;
    chunks = (g.C + cch - 1) / cch;
    const int remap = knob(kKnobXcdRemap, 1);
    const dim3 grid(remap ? xcd_grid(nb) : nb, g.B, chunks);
    if (rt.lpr * rt.rpw <= 256) {
        hipLaunchKernelGGL((bwdx_rows<NDIM, RELU, WOUT, V, U, 256>), grid, dim3(rt.lpr * rt.rpw), lds,
                           s, g, rt, cch, remap, out, gy, k, gx, pm);
    } else if constexpr (V == 4 && !(NDIM == 3 && WOUT == 2)) {
        // rows longer than 1024 voxels: up to 1024 lanes per workgroup (3D with two output
        // channels: the 18 staged rows of such a row do not fit the LDS budget, see fits())
        hipLaunchKernelGGL((bwdx_rows<NDIM, RELU, WOUT, V, U, 1024>), grid, dim3(rt.lpr * rt.rpw), lds,
                           s, g, rt, cch, remap, out, gy, k, gx, pm);
    } else {
        return hipErrorInvalidConfiguration;   // excluded by fits()
    }
    return hipGetLastError();
}

template <int NDIM, bool RELU, int WOUT, int V>
hipError_t pick_unroll(const Geom &g, const View<const float> &out, const View<const float> &gy, const float *k,
                       const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    const int u = knob(NDIM == 3 ? kKnobBwdxUnroll3d : kKnobBwdxUnroll2d, 2);
    if (u <= 2) return launch<NDIM, RELU, WOUT, V, 2>(g, out, gy, k, gx, pm, s);
    return launch<NDIM, RELU, WOUT, V, 4>(g, out, gy, k, gx, pm, s);
}

// Row fits a workgroup and its staged rows fit the LDS budget.
template <int NDIM>
bool fits(const Geom &g, int V, int wout)
{
    RowTeams rt;
    if (!make_row_teams(g, V, &rt)) return false;
    if (V < 4 && rt.lpr * rt.rpw > 256) return false;
    return staged_floats<NDIM>(rt, wout) * rt.rpw * sizeof(float) <= kMaxLds;
}

// Largest supported voxels-per-lane count not above vmax, 0 if none: V-wide
// accesses must be aligned in every view, a row must fit one workgroup and the
// staged rows the LDS budget.
template <int NDIM>
int choose_vec(const Geom &g, bool relu, int wout, int vmax, const View<const float> &out, const View<const float> &gy,
               const View<float> &gx)
{
    for (int v = 4; v >= 1; v /= 2) {
        if (v > vmax) continue;
        if (!rows_aligned(gx, g.W, v) || !rows_aligned(gy, g.W, v) || (relu && !rows_aligned(out, g.W, v))) continue;
        if (fits<NDIM>(g, v, wout)) return v;
    }
    return 0;
}

template <int NDIM, bool RELU, int WOUT>
hipError_t pick_vec(const Geom &g, const View<const float> &out, const View<const float> &gy, const float *k,
                    const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    // registers: the gathered gradient takes WOUT * K * V of them
    const int vmax = knob(NDIM == 3 ? kKnobBwdxVec3d : kKnobBwdxVec2d, NDIM == 3 ? 1 : 4);
    int v = choose_vec<NDIM>(g, RELU, WOUT, vmax, out, gy, gx);
    if (v == 0) v = choose_vec<NDIM>(g, RELU, WOUT, 4, out, gy, gx);
    if (v == 4) return pick_unroll<NDIM, RELU, WOUT, 4>(g, out, gy, k, gx, pm, s);
    if (v == 2) return pick_unroll<NDIM, RELU, WOUT, 2>(g, out, gy, k, gx, pm, s);
    if (v == 1) return pick_unroll<NDIM, RELU, WOUT, 1>(g, out, gy, k, gx, pm, s);
    return hipErrorInvalidConfiguration;   // callers check fast_backward_x_supported first
}

template <int NDIM, bool RELU>
hipError_t pick_wout(const Geom &g, const View<const float> &out, const View<const float> &gy, const float *k,
                     const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    return g.Wd == 1 ? pick_vec<NDIM, RELU, 1>(g, out, gy, k, gx, pm, s) : pick_vec<NDIM, RELU, 2>(g, out, gy, k, gx, pm, s);
}

template <int NDIM>
bool fast_backward_x_supported_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                                  const View<float> &gx)
{
    if (g.Wd > 2) return false;
    if (gx.sx != 1 || gy.sx != 1 || (relu && out.sx != 1)) return false;
    return choose_vec<NDIM>(g, relu, g.Wd, 4, out, gy, gx) != 0;
}

template <int NDIM>
hipError_t fast_backward_x_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                              const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    return relu ? pick_wout<NDIM, true>(g, out, gy, k, gx, pm, s) : pick_wout<NDIM, false>(g, out, gy, k, gx, pm, s);
}

}  // namespace bwdx
}  // namespace msd
