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

    // the first channels of grad_input are asked for before the gather: their latency passes
    // behind the gather's (lanes outside the image ask for a valid address and drop the values)
    float *gp = gx.p + (int64_t)b * gx.sb + (int64_t)z * gx.sz + (int64_t)y * gx.sy + min(x0, g.W - V);
    float first[U][V];
#pragma unroll
    for (int u = 0; u < U; u++) load_vec<V>(gp + (int64_t)min(c0 + u, c1 - 1) * gx.sc, first[u]);

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

    for (int ci = c0; ci < c1; ci += U) {
        float cur[U][V];
        int cu[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            cu[u] = min(ci + u, c1 - 1);
            if (ci == c0) {
#pragma unroll
                for (int i = 0; i < V; i++) cur[u][i] = first[u][i];
            } else {
                load_vec<V>(gp + (int64_t)cu[u] * gx.sc, cur[u]);
            }
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

// Two layers of a dense block per pass (WOUT == 2: channel 0 with the Geom's dilation and the
// weights k, channel 1 with up.d[0] and k1, both [C][K] arrays over the channels the layers
// share), with the channel loop as a software pipeline: 108 multiply-adds per voxel and channel
// leave the memory latency to be hidden by the wave itself, so the loads run kAhead steps of U
// channels ahead of the arithmetic in a ring of register sets (V floats per channel: the ring
// is small next to the gathered taps).  A set is loaded into again two steps after its
// channels were stored: overwriting the registers of stores that were only just issued would
// have to wait for them.  Nothing in the loop is under a condition: the last step repeats the
// last channel where the count is not a multiple of U (same values in, same values out), and
// the ReLU mask of the layer below comes from one load before the loop; the number of accesses
// in flight is then the same on every path and the waits are for exactly the set that is needed.
// s_waitcnt for the scalar (and LDS) counter alone: lgkmcnt(0), the vector-memory and export
// counters at their maxima
constexpr int kWaitScalarLoads = 0xC07F;
constexpr int kRingSets = 4;                     // kAhead = kRingSets - 2 steps (three to seven sets time alike)

template <int NDIM, int V, int U>
__device__ __forceinline__ void bwdx_pair_body(const Geom &g, const RowTeams &rt, int cch, int remap,
                                               const View<const float> &gy, const float *__restrict__ k,
                                               const float *__restrict__ k1, const UpperDilations &up,
                                               const View<float> &gx, const PostMask &pm)
{
    extern __shared__ float lds[];
    constexpr int WOUT = 2, K = Taps<NDIM>::K, NPQ = RowTaps<NDIM>::NPQ, NS = kRingSets;
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

    // What the channel loop starts with is asked for before the gather, so that its latency
    // passes behind the gather's (lanes outside the image ask for a valid address and drop the
    // values): the first steps of the ring, and the activation behind the pass's last channel.
    // Channels from pm.from on are outputs of the layer below: their gradient is complete with
    // this update, so its ReLU mask is applied on the way out.  (The dense block masks the one
    // channel that ends the pass; `keep` is that channel's mask.)
    const int64_t spatial = (int64_t)b * gx.sb + (int64_t)z * gx.sz + (int64_t)y * gx.sy + min(x0, g.W - V);
    float *gp = gx.p + spatial;
    float ring[NS][U][V];
    auto load_set = [&](int set, int ci) {
#pragma unroll
        for (int u = 0; u < U; u++) load_vec<V>(gp + (int64_t)min(ci + u, c1 - 1) * gx.sc, ring[set][u]);
    };
#pragma unroll
    for (int j = 0; j < NS - 2; j++) load_set(j, c0 + j * U);
    float below[V];
    load_vec<V>(pm.from < c1 ? pm.act.p + (int64_t)b * pm.act.sb + (int64_t)(c1 - 1) * pm.act.sc +
                                   (int64_t)z * pm.act.sz + (int64_t)y * pm.act.sy + min(x0, g.W - V)
                             : gp,
                below);

    float A[WOUT][K][V];
    {
        float *S = lds + (size_t)team * WOUT * NPQ * V * rt.lpr;
        float own[WOUT][NPQ][V];
        stage_source_rows<NDIM, false, WOUT, V>(g, rt, gy, gy, b, z, y, lane, act, S, own, up);
#pragma unroll
        for (int i = 0; i < V; i++) {
#pragma unroll
            for (int co = 0; co < WOUT; co++) {
                const SideTaps<V> side(x0 + i, g.W, dilation_of(g, up, co), rt.lpr);
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    side.read(S + (size_t)(co * NPQ + pq) * V * rt.lpr, A[co][pq * 3 + 0][i], A[co][pq * 3 + 2][i]);
                    A[co][pq * 3 + 1][i] = own[co][pq][i];
                }
            }
        }
    }
    if (!act) return;

    bool keep[V];
#pragma unroll
    for (int i = 0; i < V; i++) keep[i] = !(pm.from < c1) || 0.f < below[i];

    // The weights are wave-uniform: scalar loads into scalar registers, which complete in any
    // order, so a wait for some of them is a wait for all.  They are therefore asked for one
    // stage (one layer's 27 taps of one channel) ahead, into the registers of the other layer:
    // the wait before a stage's arithmetic finds its weights long since there and only has the
    // next stage's to sit out, behind 27 multiply-adds per voxel.
    typedef const __attribute__((address_space(4))) float *const_floats_t;
    const const_floats_t kw0 = (const_floats_t)(uintptr_t)k, kw1 = (const_floats_t)(uintptr_t)k1;
    float w0[K], w1[K];
    auto request = [&](const_floats_t kw, int ch, float (&w)[K]) {
#pragma unroll
        for (int t = 0; t < K; t++) w[t] = kw[(int64_t)ch * K + t];
    };
    auto finish_set = [&](int set, int ci) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int cu = min(ci + u, c1 - 1), cn = min(ci + u + 1, c1 - 1);
            float s[V];
#pragma unroll
            for (int i = 0; i < V; i++) s[i] = 0.f;
            // (the explicit wait comes before the next request on purpose: placed by the compiler
            // it would stand before the first use, behind the request, and wait for that too)
            __builtin_amdgcn_s_waitcnt(kWaitScalarLoads);
            request(kw1, cu, w1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < K; t++)
#pragma unroll
                for (int i = 0; i < V; i++) s[i] += w0[t] * A[0][t][i];
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(kWaitScalarLoads);
            request(kw0, cn, w0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < K; t++)
#pragma unroll
                for (int i = 0; i < V; i++) s[i] += w1[t] * A[1][t][i];
            const bool last = cu == c1 - 1;
#pragma unroll
            for (int i = 0; i < V; i++) {
                ring[set][u][i] += s[i];
                ring[set][u][i] = last && !keep[i] ? 0.f : ring[set][u][i];
            }
            store_vec<V>(gp + (int64_t)cu * gx.sc, ring[set][u]);
        }
    };
    request(kw0, c0, w0);
    for (int ci = c0;;) {
#pragma unroll
        for (int j = 0; j < NS; j++) {
            load_set((j + NS - 2) % NS, ci + (NS - 2) * U);
            __builtin_amdgcn_sched_barrier(0);   // (the loads stay ahead of the arithmetic)
            finish_set(j, ci);
            ci += U;
            if (ci >= c1) return;
        }
    }
}

constexpr size_t kMaxLdsOneChannel = 64 * 1024;

// One input channel, one output channel (the step of the dense block's chain in which the upper
// layer of a pair finishes the channel the lower layer wrote): there is no channel loop to keep
// the gathered taps for, so they are multiplied as they are read from the staged rows and a
// lane can own four voxels at 80 registers: a quarter of the workgroups (128^3: 20 against 24
// us with the general kernel; what remains is one launch and one chain of round trips: gather,
// LDS, store; one, two or four voxels per lane time alike).
template <int NDIM, int V>
__global__ __launch_bounds__(256, 6) void bwdx_one_channel(Geom g, RowTeams rt, int remap, View<const float> gy,
                                                           const float *__restrict__ k, View<float> gx, PostMask pm)
{
    extern __shared__ float lds[];
    constexpr int NPQ = RowTaps<NDIM>::NPQ;
    const int team = threadIdx.x / rt.lpr, lane = threadIdx.x % rt.lpr;
    const int lb = block_for_xcd(blockIdx.x, gridDim.x, remap);
    if (lb * rt.rpw >= rt.nrows) return;   // padding block (whole workgroup)
    const int row = lb * rt.rpw + team;
    const int x0 = lane * V;
    const bool act = row < rt.nrows && x0 < g.W;
    const int rr = min(row, rt.nrows - 1);
    const int y = rr % g.H, z = rr / g.H;
    const int b = blockIdx.y;
    // the channel's own values and its activation are asked for before the gather
    const int64_t at = (int64_t)b * gx.sb + (int64_t)z * gx.sz + (int64_t)y * gx.sy + min(x0, g.W - V);
    float cur[V], below[V];
    load_vec<V>(gx.p + at, cur);
    const bool masked = pm.from < 1;
    load_vec<V>(masked ? pm.act.p + (int64_t)b * pm.act.sb + (int64_t)z * pm.act.sz + (int64_t)y * pm.act.sy +
                             min(x0, g.W - V)
                       : gx.p + at,
                below);
    float *S = lds + (size_t)team * NPQ * V * rt.lpr;
    float own[1][NPQ][V];
    stage_source_rows<NDIM, false, 1, V>(g, rt, gy, gy, b, z, y, lane, act, S, own);
    if (!act) return;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const SideTaps<V> side(x0 + i, g.W, g.dil, rt.lpr);
        float s = 0.f;
#pragma unroll
        for (int pq = 0; pq < NPQ; pq++) {
            float t0, t2;
            side.read(S + (size_t)pq * V * rt.lpr, t0, t2);
            s += k[pq * 3 + 0] * t0;
            s += k[pq * 3 + 1] * own[0][pq][i];
            s += k[pq * 3 + 2] * t2;
        }
        cur[i] += s;
        cur[i] = masked && !(0.f < below[i]) ? 0.f : cur[i];
    }
    store_vec<V>(gx.p + at, cur);
}

template <int NDIM>
int one_channel_vec(const Geom &g, const View<const float> &gy, const View<float> &gx, const PostMask &pm)
{
    if (g.C != 1 || g.Wd != 1 || gx.sx != 1 || gy.sx != 1 || (pm.from < 1 && pm.act.sx != 1)) return 0;
    for (int v = 4; v >= 1; v /= 2) {
        if (!rows_aligned(gx, g.W, v) || !rows_aligned(gy, g.W, v) || (pm.from < 1 && !rows_aligned(pm.act, g.W, v)))
            continue;
        RowTeams rt;
        if (!make_row_teams(g, v, &rt) || rt.lpr * rt.rpw > 256) continue;
        if (staged_floats<NDIM>(rt, 1) * rt.rpw * sizeof(float) <= kMaxLdsOneChannel) return v;
    }
    return 0;
}

template <int NDIM>
hipError_t one_channel_nd(const Geom &g, const View<const float> &gy, const float *k, const View<float> &gx,
                          const PostMask &pm, hipStream_t s)
{
    const int v = one_channel_vec<NDIM>(g, gy, gx, pm);
    if (v == 0) return hipErrorInvalidConfiguration;
    RowTeams rt;
    make_row_teams(g, v, &rt);
    const int nb = (rt.nrows + rt.rpw - 1) / rt.rpw;
    const size_t lds = staged_floats<NDIM>(rt, 1) * rt.rpw * sizeof(float);
    const int remap = knob(kKnobXcdRemap, 1);
    const dim3 grid(remap ? xcd_grid(nb) : nb, g.B, 1), block(rt.lpr * rt.rpw);
    if (v == 4)
        hipLaunchKernelGGL((bwdx_one_channel<NDIM, 4>), grid, block, lds, s, g, rt, remap, gy, k, gx, pm);
    else if (v == 2)
        hipLaunchKernelGGL((bwdx_one_channel<NDIM, 2>), grid, block, lds, s, g, rt, remap, gy, k, gx, pm);
    else
        hipLaunchKernelGGL((bwdx_one_channel<NDIM, 1>), grid, block, lds, s, g, rt, remap, gy, k, gx, pm);
    return hipGetLastError();
}

constexpr size_t kMaxLds = 64 * 1024;

template <int NDIM, bool RELU, int WOUT, int V, int U, int MAXT>
__global__ __launch_bounds__(MAXT) void bwdx_rows(Geom g, RowTeams rt, int cch, int remap, View<const float> out,
                                                  View<const float> gy, const float *__restrict__ k, View<float> gx,
                                                  PostMask pm)
{
    bwdx_rows_body<NDIM, RELU, WOUT, V, U>(g, rt, cch, remap, out, gy, k, gx, pm);
}

template <int NDIM, int V, int U>
__global__ __launch_bounds__(256) void bwdx_rows_pair(Geom g, RowTeams rt, int cch, int remap, View<const float> gy,
                                                      const float *__restrict__ k, const float *__restrict__ k1,
                                                      UpperDilations up, View<float> gx, PostMask pm)
{
    bwdx_pair_body<NDIM, V, U>(g, rt, cch, remap, gy, k, k1, up, gx, pm);
}

template <int NDIM, bool RELU, int WOUT, int V, int U, bool PAIR = false>
hipError_t launch(const Geom &g, const View<const float> &out, const View<const float> &gy, const float *k,
                  const View<float> &gx, const PostMask &pm, hipStream_t s, const float *k1 = nullptr,
                  const UpperDilations up = UpperDilations{{0, 0}})
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
    if constexpr (PAIR) {
        if (rt.lpr * rt.rpw > 256) return hipErrorInvalidConfiguration;   // excluded by pair_supported()
        hipLaunchKernelGGL((bwdx_rows_pair<NDIM, V, U>), grid, dim3(rt.lpr * rt.rpw), lds, s, g, rt, cch, remap, gy, k,
                           k1, up, gx, pm);
        return hipGetLastError();
    }
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

// Two layers of a dense block (one output channel each) over the g.C input channels they
// share: g.dil and k are the lower layer's, group->dil[1] and group->k_up[0] the upper one's;
// gy holds the two masked output gradients as consecutive channels (lower first).
template <int NDIM>
int pair_vec(const Geom &g, const View<const float> &gy, const View<float> &gx)
{
    if (g.Wd != 2 || gx.sx != 1 || gy.sx != 1) return 0;
    const int vmax = knob(NDIM == 3 ? kKnobBwdxVec3d : kKnobBwdxVec2d, NDIM == 3 ? 1 : 4);
    // (two voxels per lane at most: four would hold 216 gathered values per lane)
    for (int pass = 0; pass < 2; pass++)
        for (int v = 2; v >= 1; v /= 2) {
            if (pass == 0 && v > vmax) continue;
            if (!rows_aligned(gx, g.W, v) || !rows_aligned(gy, g.W, v) || !fits<NDIM>(g, v, 2)) continue;
            RowTeams rt;
            make_row_teams(g, v, &rt);
            if (rt.lpr * rt.rpw <= 256) return v;
        }
    return 0;
}

template <int NDIM, int V>
hipError_t pair_unroll(const Geom &g, const View<const float> &gy, const float *k, const View<float> &gx,
                       const PostMask &pm, hipStream_t s, const float *k1, const UpperDilations up)
{
    const int u = knob(NDIM == 3 ? kKnobBwdxUnroll3d : kKnobBwdxUnroll2d, 2);
    if (u <= 2) return launch<NDIM, false, 2, V, 2, true>(g, gy, gy, k, gx, pm, s, k1, up);
    return launch<NDIM, false, 2, V, 4, true>(g, gy, gy, k, gx, pm, s, k1, up);
}

template <int NDIM>
hipError_t pair_nd(const Geom &g, const View<const float> &gy, const float *k, const View<float> &gx, const PostMask &pm,
                   hipStream_t s, const LayerGroup *group)
{
    if (!group || group->n != 2 || !group->k_up[0]) return hipErrorInvalidValue;
    if (pm.from < g.C - 1) return hipErrorInvalidValue;   // (at most the channel that ends the pass is masked)
    Geom g2 = g;
    g2.dil = group->dil[0];
    const UpperDilations up{{group->dil[1], 0}};
    const int v = pair_vec<NDIM>(g2, gy, gx);
    if (v == 2) return pair_unroll<NDIM, 2>(g2, gy, k, gx, pm, s, group->k_up[0], up);
    if (v == 1) return pair_unroll<NDIM, 1>(g2, gy, k, gx, pm, s, group->k_up[0], up);
    return hipErrorInvalidConfiguration;
}

template <int NDIM>
hipError_t fast_backward_x_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                              const float *k, const View<float> &gx, const PostMask &pm, hipStream_t s)
{
    return relu ? pick_wout<NDIM, true>(g, out, gy, k, gx, pm, s) : pick_wout<NDIM, false>(g, out, gy, k, gx, pm, s);
}

}  // namespace bwdx
}  // namespace msd
