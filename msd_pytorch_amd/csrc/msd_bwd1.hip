// Backward pass of one layer (or of two layers at once) over ONE input channel, 2D, fp32:
// grad_input of that channel, the nine weight gradients of that channel per layer, and the
// channel's ReLU mask on the way out.
//
// The dense block's backward loop takes its layers two or three at a time (msd_api.hip): the
// upper layers of such a group first have to finish the gradients of the channels the lower
// layers wrote, one channel at a time out of up to a hundred.  The fused kernel (msd_bwdxk_impl.h) does that too, but its
// pipeline of 16-channel blocks on the matrix cores runs in full for the one channel (20 us at
// 1024 x 1024); here the channel is four planes of memory traffic and 18 multiply-adds per
// voxel on the vector pipe: the gather of msd_rows.h (the same one, so the same values), one
// load of x and grad_input per lane, nine running sums per lane for the weight gradient,
// reduced once per workgroup into a row of partial sums (fixed order; second pass as for the
// other weight-gradient kernels).
// Semantics: conv2d_backward_x.cu:109-208 and conv2d_backward_k.cu:61-112 of the reference,
// restricted to one input channel.
#include "msd_kernels.h"
#include "msd_rows.h"

namespace msd {
namespace bwd1 {

constexpr int kThreads = 256;
constexpr int K = 9, NPQ = 3;

struct Args {
    Geom g;
    RowTeams rt;
    int ngroups, total_groups, tiles_per_wg;
    int masked;
    int gy_sb, gy_sc, gy_sy, x_sb, x_sy, gx_sb, gx_sy;
    UpperDilations up;   // the second layer's dilation where it has its own
};

// WOUT layers (output gradients in consecutive channels of gy, weights kw and kw1).
template <int V, int WOUT>
__global__ __launch_bounds__(kThreads, 4) void bwd_one_channel(const Args a, const float *__restrict__ gyp,
                                                            const float *__restrict__ xp, float *__restrict__ gxp,
                                                            const float *__restrict__ actp,
                                                            const float *__restrict__ kw,
                                                            const float *__restrict__ kw1, float *__restrict__ part)
{
    extern __shared__ float lds[];
    constexpr int KR = WOUT * K;
    const Geom &g = a.g;
    const RowTeams &rt = a.rt;
    const int tid = threadIdx.x;
    const int team = tid / rt.lpr, lane0 = tid % rt.lpr;
    float w[KR];
#pragma unroll
    for (int t = 0; t < KR; t++) w[t] = t < K ? kw[t] : kw1[t - K];     // uniform: scalar loads
    float ksum[KR];
#pragma unroll
    for (int t = 0; t < KR; t++) ksum[t] = 0.f;
    const View<const float> none{nullptr, 0, 0, 0, 0, 0};
    const View<const float> gyv{gyp, a.gy_sb, a.gy_sc, 0, a.gy_sy, 1};

    for (int ti = 0; ti < a.tiles_per_wg; ti++) {
        const int grp = blockIdx.x + ti * gridDim.x;          // uniform
        if (grp >= a.total_groups) break;
        // what depends on the lane only is computed per tile on purpose (the lane number passes
        // through an empty asm): hoisted out of the loop, the LDS positions of all the taps
        // would occupy a hundred registers for a loop that mostly runs once
        int lane = lane0;
        asm volatile("" : "+v"(lane));
        float *S = lds + (size_t)team * WOUT * NPQ * V * rt.lpr;
        const int x0 = lane * V;
        const int xc = min(x0, g.W - V);
        const int gi = grp % a.ngroups, b = grp / a.ngroups;
        const int row = gi * rt.rpw + team;
        const bool rowok = row < g.H;
        const int y = rowok ? row : g.H - 1;
        const bool act = rowok && x0 < g.W;
        // the channel's own values are asked for first: their latency passes behind the gather
        const int64_t xo = (int64_t)b * a.x_sb + (int64_t)y * a.x_sy + xc;
        const int64_t go = (int64_t)b * a.gx_sb + (int64_t)y * a.gx_sy + xc;
        float xv[V], gv[V], m[V];
        load_vec<V>(xp + xo, xv);
        load_vec<V>(gxp + go, gv);
        if (a.masked) load_vec<V>(actp + go, m);   // uniform; the activations share grad_input's layout
        float own[WOUT][NPQ][V];
        stage_source_rows<2, false, WOUT, V>(g, rt, none, gyv, b, 0, y, lane, act, S, own, a.up);
        // lanes outside the image take their side taps from the last voxel's positions: their x counts as zero
#pragma unroll
        for (int i = 0; i < V; i++) xv[i] = act ? xv[i] : 0.f;
        // layer by layer, so that only one layer's nine taps per voxel are live at a time
#pragma unroll
        for (int co = 0; co < WOUT; co++) {
            // voxel by voxel: the twelve LDS reads of a voxel together, then its sums (the
            // scheduling barriers keep the reads of the other voxels out of its registers)
#pragma unroll
            for (int i = 0; i < V; i++) {
                const SideTaps<V> side(min(x0 + i, g.W - 1), g.W, dilation_of(g, a.up, co), rt.lpr);
                float ra[NPQ][4];
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    const float *srow = S + (size_t)(co * NPQ + pq) * V * rt.lpr;
                    ra[pq][0] = srow[side.i0a];
                    ra[pq][1] = srow[side.i0b];
                    ra[pq][2] = srow[side.i2a];
                    ra[pq][3] = srow[side.i2b];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    const float t[3] = {(side.m0a ? ra[pq][0] : 0.f) + (side.m0b ? ra[pq][1] : 0.f), own[co][pq][i],
                                        (side.m2a ? ra[pq][2] : 0.f) + (side.m2b ? ra[pq][3] : 0.f)};
#pragma unroll
                    for (int q = 0; q < 3; q++) {
                        gv[i] += w[co * K + pq * 3 + q] * t[q];
                        ksum[co * K + pq * 3 + q] += t[q] * xv[i];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (a.masked) {
#pragma unroll
            for (int i = 0; i < V; i++) gv[i] = 0.f < m[i] ? gv[i] : 0.f;
        }
        if (act) store_vec<V>(gxp + go, gv);
        __syncthreads();                          // the next tile overwrites the staged rows
    }

    // the lanes of a wave by a fixed shuffle tree, then the waves in order
    const int wave = tid / kWave, wl = tid % kWave, nwaves = blockDim.x / kWave;
#pragma unroll
    for (int t = 0; t < KR; t++) {
        float s = ksum[t];
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_down(s, off, kWave);
        if (wl == 0) lds[wave * KR + t] = s;
    }
    __syncthreads();
    if (tid < KR) {                               // column = layer * 9 + tap
        float s = 0.f;
        for (int v = 0; v < nwaves; v++) s += lds[v * KR + tid];
        part[(int64_t)tid * kMaxPartialRows + blockIdx.x] = s;
    }
}

// Voxels per lane, or 0: rows of whole waves that one team of at most 256 lanes covers,
// naturally aligned V-wide accesses in all three tensors.
// Two layers come with a pass of three layers over the other channels, which takes rows of whole
// groups of four voxels only: such rows never need one voxel per lane.
inline int min_vec(const Geom &g) { return g.Wd == 2 ? 2 : 1; }

int choose_vec(const Geom &g, const View<const float> &gy, const View<const float> &x, const View<float> &gx,
               RowTeams *rt)
{
    for (int v = 4; v >= min_vec(g); v /= 2) {
        if (!rows_aligned(gy, g.W, v) || !rows_aligned(x, g.W, v) || !rows_aligned(gx, g.W, v)) continue;
        if (!make_row_teams(g, v, rt)) continue;
        if (rt->lpr % kWave != 0 || rt->lpr * rt->rpw > kThreads) continue;
        return v;
    }
    return 0;
}

bool in_range(const Geom &g, const View<const float> &v)
{
    const int64_t lim = (int64_t)1 << 31;
    return v.sx == 1 && v.sb < lim && v.sc < lim && v.sy < lim && (int64_t)(g.H - 1) * v.sy + g.W < lim;
}

}  // namespace bwd1

bool fast_backward_one_channel_supported_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                            const View<float> &gx)
{
    if (g.ndim != 2 || g.C != 1 || (g.Wd != 1 && g.Wd != 2) || g.D != 1) return false;
    const View<const float> gxc{gx.p, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
    if (!bwd1::in_range(g, gy) || !bwd1::in_range(g, x) || !bwd1::in_range(g, gxc)) return false;
    RowTeams rt;
    return bwd1::choose_vec(g, gy, x, gx, &rt) != 0;
}

template <int WOUT>
static void launch_one_channel(int v, dim3 grid, dim3 block, size_t lds, hipStream_t s, const bwd1::Args &a,
                               const float *gy, const float *x, float *gx, const float *act, const float *k,
                               const float *k1, float *part)
{
    if (v == 4)
        hipLaunchKernelGGL((bwd1::bwd_one_channel<4, WOUT>), grid, block, lds, s, a, gy, x, gx, act, k, k1, part);
    else if (v == 2)
        hipLaunchKernelGGL((bwd1::bwd_one_channel<2, WOUT>), grid, block, lds, s, a, gy, x, gx, act, k, k1, part);
    else if constexpr (WOUT == 1)     // (two layers: see min_vec)
        hipLaunchKernelGGL((bwd1::bwd_one_channel<1, WOUT>), grid, block, lds, s, a, gy, x, gx, act, k, k1, part);
}

hipError_t fast_backward_one_channel_2d(const Geom &g, const View<const float> &gy, const View<const float> &x,
                                        const float *k, const View<float> &gx, const PostMask &pm, float *gk,
                                        float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group)
{
    if (g.Wd != 1 && g.Wd != 2) return hipErrorInvalidValue;
    if (group && (group->n != 2 || g.Wd != 2)) return hipErrorInvalidValue;
    bwd1::Args a;
    a.g = g;
    a.up = UpperDilations{{0, 0}};
    if (group) {
        a.g.dil = group->dil[0];
        a.up.d[0] = group->dil[1];
    }
    const int v = bwd1::choose_vec(g, gy, x, gx, &a.rt);
    if (v == 0) return hipErrorInvalidConfiguration;
    a.ngroups = (g.H + a.rt.rpw - 1) / a.rt.rpw;
    const int64_t total = (int64_t)a.ngroups * g.B;
    if (total > INT32_MAX) return hipErrorInvalidConfiguration;
    a.total_groups = (int)total;
    const int wgs = (int)std::min<int64_t>(total, kMaxPartialRows);
    a.tiles_per_wg = (int)((total + wgs - 1) / wgs);
    a.masked = pm.from < g.C;
    a.gy_sb = (int)gy.sb; a.gy_sc = (int)gy.sc; a.gy_sy = (int)gy.sy;
    a.x_sb = (int)x.sb; a.x_sy = (int)x.sy;
    a.gx_sb = (int)gx.sb; a.gx_sy = (int)gx.sy;
    const float *actp = a.masked ? pm.act.p : x.p;
    float *part = defer ? const_cast<float *>(defer->part) : ws + backward_k_mask_floats(g);
    const size_t lds = std::max((size_t)a.rt.rpw * g.Wd * bwd1::NPQ * v * a.rt.lpr,
                                (size_t)(bwd1::kThreads / kWave) * g.Wd * bwd1::K) * sizeof(float);
    const dim3 grid(wgs), block(a.rt.lpr * a.rt.rpw);
    // the second layer's weights follow the first's, or are another layer's
    const float *k1 = group ? group->k_up[0] : k + bwd1::K;
    if (g.Wd == 2)
        launch_one_channel<2>(v, grid, block, lds, s, a, gy.p, x.p, gx.p, actp, k, k1, part);
    else
        launch_one_channel<1>(v, grid, block, lds, s, a, gy.p, x.p, gx.p, actp, k, k1, part);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nk = (int64_t)g.Wd * bwd1::K;
    const ReduceJob job{part, gk, nullptr, nk, nk, wgs, {group ? group->gk_up[0] : nullptr, nullptr},
                        group ? (int64_t)bwd1::K : nk, group ? (int64_t)bwd1::K : nk};
    if (defer) {
        *defer = job;
        return hipSuccess;
    }
    return reduce_columns_batch(&job, 1, s);
}

}  // namespace msd
