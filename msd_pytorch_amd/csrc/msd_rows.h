// Row-team mapping and LDS-staged adjoint gather shared by the specialised
// fp32 backward kernels.
//
// A workgroup is split into teams of `lpr` lanes; a team owns one image row
// (z, y) and each lane V consecutive voxels of it.  lpr is a power of two below
// a wavefront or a multiple of 64, so a wave never holds lanes of a row it
// shares with another wave only in part.
//
// Adjoint gather.  For input voxel u and weight tap t = (p, q, r),
//     A[t](u) = sum of m(v) over the output voxels v whose tap t reads u,
// m being the output gradient, masked by [0 < output] when RELU.  Along z and y
// the sources of a whole row are whole rows (one, or two when the fold of the
// symmetric padding maps a second row onto it); they are summed while they are
// staged into LDS:  S[p][q][x] = sum of m over the source rows of (p, q).
// Along x each voxel then takes at most two values of S per tap (the second
// again from the fold), read from LDS with clamped indices and select masks, so
// the code is free of divergent branches.
//
// LDS layout of one staged row: element x lives at (x % V) * lpr + x / V, which
// makes both the V-wide writes and the shifted or mirrored reads of a team hit
// consecutive banks.
#pragma once

#include "msd_adjoint.h"

namespace msd {

struct RowTeams {
    int V;       // voxels per lane
    int lpr;     // lanes per row (per segment of a row that is cut into segments)
    int rpw;     // rows (teams) per workgroup
    int nrows;   // D * H
};

struct RowSegments {
    int segs;    // segments a row is cut into (1: a team owns a whole row)
    int halo;    // floats appended to each staged row for the neighbours of a segment (0 when segs == 1)
};

constexpr int kSegmentLanes = 256;   // lanes of a team that owns a segment of a long row

// With `sg`: rows longer than kSegmentLanes * V voxels are cut into segments of that length
// (the last one may be shorter), one team (and workgroup) each; the kernels that ask for it
// stage a halo of `dil` values on either side (stage_source_segment).  dil <= 128.
inline bool make_row_teams(const Geom &g, int V, RowTeams *rt, RowSegments *sg = nullptr)
{
    const int need = (g.W + V - 1) / V;
    int lpr;
    if (need <= kWave) {
        lpr = 1;
        while (lpr < need) lpr *= 2;
    } else {
        lpr = (need + kWave - 1) / kWave * kWave;
    }
    rt->V = V;
    rt->nrows = g.D * g.H;
    if (sg) *sg = RowSegments{1, 0};
    if (sg && lpr > kSegmentLanes) {
        const int segw = kSegmentLanes * V;
        if (2 * g.dil > kSegmentLanes) return false;
        rt->lpr = kSegmentLanes;
        rt->rpw = 1;
        sg->segs = (g.W + segw - 1) / segw;
        sg->halo = (2 * g.dil + 3) & ~3;         // keeps what follows the staged rows 16-byte aligned
        return true;
    }
    if (lpr > 1024) return false;
    rt->lpr = lpr;
    rt->rpw = lpr >= 256 ? 1 : 256 / lpr;
    return true;
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// V consecutive floats as one naturally aligned 4-, 8- or 16-byte access.
template <int V> __device__ __forceinline__ void load_vec(const float *p, float (&d)[V]);
template <> __device__ __forceinline__ void load_vec<1>(const float *p, float (&d)[1]) { d[0] = *p; }
template <> __device__ __forceinline__ void load_vec<2>(const float *p, float (&d)[2])
{
    const f32x2 v = *reinterpret_cast<const f32x2 *>(p);
    d[0] = v[0]; d[1] = v[1];
}
template <> __device__ __forceinline__ void load_vec<4>(const float *p, float (&d)[4])
{
    const f32x4 v = *reinterpret_cast<const f32x4 *>(p);
    d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
}
// The same from global memory at a wave-uniform 64-bit base plus a 32-bit byte offset per
// lane: the form the load instruction takes directly (scalar base, vector offset).
template <int V>
__device__ __forceinline__ void load_global_vec(uint64_t base, uint32_t byte_offset, float (&d)[V])
{
    typedef const __attribute__((address_space(1))) char *gbytes_t;
    gbytes_t p = reinterpret_cast<gbytes_t>(base) + byte_offset;
    if constexpr (V == 1) {
        d[0] = *reinterpret_cast<const __attribute__((address_space(1))) float *>(p);
    } else {
        typedef float vec_t __attribute__((ext_vector_type(V)));
        const vec_t v = *reinterpret_cast<const __attribute__((address_space(1))) vec_t *>(p);
#pragma unroll
        for (int i = 0; i < V; i++) d[i] = v[i];
    }
}
// Four consecutive floats at an address that is only known to be a multiple of four bytes.
__device__ __forceinline__ void load_global_vec4_unaligned(uint64_t base, uint32_t byte_offset, float (&d)[4])
{
    typedef float vec_t __attribute__((ext_vector_type(4), aligned(4)));
    typedef const __attribute__((address_space(1))) char *gbytes_t;
    gbytes_t p = reinterpret_cast<gbytes_t>(base) + byte_offset;
    const vec_t v = *reinterpret_cast<const __attribute__((address_space(1))) vec_t *>(p);
#pragma unroll
    for (int i = 0; i < 4; i++) d[i] = v[i];
}
template <int V>
__device__ __forceinline__ void store_global_vec(uint64_t base, uint32_t byte_offset, const float (&d)[V])
{
    typedef __attribute__((address_space(1))) char *gbytes_t;
    gbytes_t p = reinterpret_cast<gbytes_t>(base) + byte_offset;
    if constexpr (V == 1) {
        *reinterpret_cast<__attribute__((address_space(1))) float *>(p) = d[0];
    } else {
        typedef float vec_t __attribute__((ext_vector_type(V)));
        vec_t v;
#pragma unroll
        for (int i = 0; i < V; i++) v[i] = d[i];
        *reinterpret_cast<__attribute__((address_space(1))) vec_t *>(p) = v;
    }
}
template <int V> __device__ __forceinline__ void store_vec(float *p, const float (&d)[V]);
template <> __device__ __forceinline__ void store_vec<1>(float *p, const float (&d)[1]) { *p = d[0]; }
template <> __device__ __forceinline__ void store_vec<2>(float *p, const float (&d)[2])
{
    f32x2 v = {d[0], d[1]};
    *reinterpret_cast<f32x2 *>(p) = v;
}
template <> __device__ __forceinline__ void store_vec<4>(float *p, const float (&d)[4])
{
    f32x4 v = {d[0], d[1], d[2], d[3]};
    *reinterpret_cast<f32x4 *>(p) = v;
}

// True when V-wide accesses at multiples of V along x are naturally aligned
// for every row of the view.
template <typename T>
inline bool rows_aligned(const View<T> &v, int W, int V)
{
    if (V == 1) return true;
    return W % V == 0 && v.sb % V == 0 && v.sc % V == 0 && v.sz % V == 0 && v.sy % V == 0 &&
           reinterpret_cast<uintptr_t>(v.p) % (V * sizeof(float)) == 0;
}

template <int NDIM> struct RowTaps { static constexpr int NPQ = NDIM == 3 ? 9 : 3; };

// Floats of LDS one team needs for `wout` output channels.
template <int NDIM>
inline size_t staged_floats(const RowTeams &rt, int wout)
{
    return (size_t)wout * RowTaps<NDIM>::NPQ * rt.V * rt.lpr;
}

// Dilations of the output channels above the first where they have one of their own (two or
// three layers of a dense block gathered in one pass); 0: the layer's dilation.
struct UpperDilations {
    int d[2];
};
__device__ __forceinline__ int dilation_of(const Geom &g, const UpperDilations &up, int co)
{
    return (co >= 1 && co <= 2 && up.d[co - 1] > 0) ? up.d[co - 1] : g.dil;
}

// Stage S[co][pq] of the team's row into LDS (see the header comment) and keep
// the lane's own V values of every staged row in `own`.  Every lane of the
// workgroup must call this; lanes outside the image (`act` false) stage zeros.
// Ends with a workgroup barrier.
// `up`: the dilations of the output channels that have one of their own.
template <int NDIM, bool RELU, int WOUT, int V>
__device__ __forceinline__ void stage_source_rows(const Geom &g, const RowTeams &rt, const View<const float> &out,
                                                  const View<const float> &gy, int b, int z, int y, int lane,
                                                  bool act, float *__restrict__ S,
                                                  float (&own)[WOUT][RowTaps<NDIM>::NPQ][V],
                                                  const UpperDilations up = UpperDilations{{0, 0}})
{
    constexpr int NZ = Taps<NDIM>::NZ, NPQ = RowTaps<NDIM>::NPQ;
    const int x0 = min(lane * V, g.W - V);   // lanes past the row read a valid address; their values are dropped
#pragma unroll
    for (int co = 0; co < WOUT; co++) {
        const int dil = dilation_of(g, up, co);
        const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
        const AxisSources sy = adjoint_sources(y, g.H, dil);
        // rows whose taps fold: within dil of a y (or z) border
        const bool folds = y < dil || y + dil >= g.H || (NDIM == 3 && (z < dil || z + dil >= g.D));
        const float *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc + x0;
        const float *oc = RELU ? out.p + (int64_t)b * out.sb + (int64_t)co * out.sc + x0 : nullptr;
        float s[NPQ][V];
        // One masked source row, loaded from a clamped (always valid) address
        // and zeroed afterwards if it does not count: no branch around the
        // loads, so all of them are in flight together.
        auto add_row = [&](int pq, int cz, int cy, bool ok, bool first) {
            cz = min(max(cz, 0), g.D - 1);
            cy = min(max(cy, 0), g.H - 1);
            float m[V];
            load_vec<V>(gc + (int64_t)cz * gy.sz + (int64_t)cy * gy.sy, m);
            if (RELU) {
                float o[V];
                load_vec<V>(oc + (int64_t)cz * out.sz + (int64_t)cy * out.sy, o);
#pragma unroll
                for (int i = 0; i < V; i++) m[i] = 0.f < o[i] ? m[i] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < V; i++) s[pq][i] = (first ? 0.f : s[pq][i]) + (ok && act ? m[i] : 0.f);
        };
#pragma unroll
        for (int p = 0; p < NZ; p++)
#pragma unroll
            for (int q = 0; q < 3; q++)
                add_row(p * 3 + q, sz.c[p][0], sy.c[q][0], sz.ok[p][0] && sy.ok[q][0], true);
        if (folds) {
#pragma unroll
            for (int p = 0; p < NZ; p++)
#pragma unroll
                for (int q = 0; q < 3; q++) {
                    add_row(p * 3 + q, sz.c[p][0], sy.c[q][1], sz.ok[p][0] && sy.ok[q][1], false);
                    if (NDIM == 3) {
                        add_row(p * 3 + q, sz.c[p][1], sy.c[q][0], sz.ok[p][1] && sy.ok[q][0], false);
                        add_row(p * 3 + q, sz.c[p][1], sy.c[q][1], sz.ok[p][1] && sy.ok[q][1], false);
                    }
                }
        }
#pragma unroll
        for (int pq = 0; pq < NPQ; pq++) {
            float *row = S + (size_t)(co * NPQ + pq) * V * rt.lpr;
#pragma unroll
            for (int i = 0; i < V; i++) {
                own[co][pq][i] = s[pq][i];
                row[i * rt.lpr + lane] = s[pq][i];
            }
        }
    }
    __syncthreads();
}

// stage_source_rows (no ReLU mask) in two steps, so that a kernel can ask for the next tile's
// rows while it still works on the current tile: request_source_rows only issues the loads of
// the first source row of every (co, p, q) (clamped, always valid addresses; nothing else is
// done with the values), finish_source_rows applies the masks, adds the second and further
// source rows of the rows that fold, stages the sums and ends with a workgroup barrier.
template <int NDIM, int WOUT, int V>
__device__ __forceinline__ void request_source_rows(const Geom &g, const View<const float> &gy, int b, int z, int y,
                                                    int lane, float (&m)[WOUT][RowTaps<NDIM>::NPQ][V],
                                                    const UpperDilations up = UpperDilations{{0, 0}})
{
    constexpr int NZ = Taps<NDIM>::NZ;
    const int x0 = min(lane * V, g.W - V);
#pragma unroll
    for (int co = 0; co < WOUT; co++) {
        const int dil = dilation_of(g, up, co);
        const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
        const AxisSources sy = adjoint_sources(y, g.H, dil);
        const float *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc + x0;
#pragma unroll
        for (int p = 0; p < NZ; p++)
#pragma unroll
            for (int q = 0; q < 3; q++) {
                const int cz = min(max(sz.c[p][0], 0), g.D - 1), cy = min(max(sy.c[q][0], 0), g.H - 1);
                load_vec<V>(gc + (int64_t)cz * gy.sz + (int64_t)cy * gy.sy, m[co][p * 3 + q]);
            }
    }
}

template <int NDIM, int WOUT, int V>
__device__ __forceinline__ void finish_source_rows(const Geom &g, const RowTeams &rt, const View<const float> &gy, int b,
                                                   int z, int y, int lane, bool act, float *__restrict__ S,
                                                   const float (&m)[WOUT][RowTaps<NDIM>::NPQ][V],
                                                   float (&own)[WOUT][RowTaps<NDIM>::NPQ][V],
                                                   const UpperDilations up = UpperDilations{{0, 0}})
{
    constexpr int NZ = Taps<NDIM>::NZ, NPQ = RowTaps<NDIM>::NPQ;
    const int x0 = min(lane * V, g.W - V);
    float s[WOUT][NPQ][V];
    bool any_folds = false;
#pragma unroll
    for (int co = 0; co < WOUT; co++) {
        const int dil = dilation_of(g, up, co);
        const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
        const AxisSources sy = adjoint_sources(y, g.H, dil);
        any_folds = any_folds || y < dil || y + dil >= g.H || (NDIM == 3 && (z < dil || z + dil >= g.D));
#pragma unroll
        for (int p = 0; p < NZ; p++)
#pragma unroll
            for (int q = 0; q < 3; q++)
#pragma unroll
                for (int i = 0; i < V; i++)
                    s[co][p * 3 + q][i] = sz.ok[p][0] && sy.ok[q][0] && act ? m[co][p * 3 + q][i] : 0.f;
    }
    if (any_folds) {
        // rows within dil of a y (or z) border: the other source rows of every output channel,
        // all requested before the first is used
        float e[WOUT][NPQ][NDIM == 3 ? 3 : 1][V];
#pragma unroll
        for (int co = 0; co < WOUT; co++) {
            const int dil = dilation_of(g, up, co);
            const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
            const AxisSources sy = adjoint_sources(y, g.H, dil);
            const float *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc + x0;
            auto row = [&](int cz, int cy, float (&d)[V]) {
                cz = min(max(cz, 0), g.D - 1);
                cy = min(max(cy, 0), g.H - 1);
                load_vec<V>(gc + (int64_t)cz * gy.sz + (int64_t)cy * gy.sy, d);
            };
#pragma unroll
            for (int p = 0; p < NZ; p++)
#pragma unroll
                for (int q = 0; q < 3; q++) {
                    row(sz.c[p][0], sy.c[q][1], e[co][p * 3 + q][0]);
                    if (NDIM == 3) {
                        row(sz.c[p][1], sy.c[q][0], e[co][p * 3 + q][1]);
                        row(sz.c[p][1], sy.c[q][1], e[co][p * 3 + q][2]);
                    }
                }
        }
#pragma unroll
        for (int co = 0; co < WOUT; co++) {
            const int dil = dilation_of(g, up, co);
            const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
            const AxisSources sy = adjoint_sources(y, g.H, dil);
#pragma unroll
            for (int p = 0; p < NZ; p++)
#pragma unroll
                for (int q = 0; q < 3; q++)
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        // (the same order of additions as stage_source_rows)
                        s[co][p * 3 + q][i] += sz.ok[p][0] && sy.ok[q][1] && act ? e[co][p * 3 + q][0][i] : 0.f;
                        if (NDIM == 3) {
                            s[co][p * 3 + q][i] += sz.ok[p][1] && sy.ok[q][0] && act ? e[co][p * 3 + q][1][i] : 0.f;
                            s[co][p * 3 + q][i] += sz.ok[p][1] && sy.ok[q][1] && act ? e[co][p * 3 + q][2][i] : 0.f;
                        }
                    }
        }
    }
#pragma unroll
    for (int co = 0; co < WOUT; co++)
#pragma unroll
        for (int pq = 0; pq < NPQ; pq++) {
            float *row = S + (size_t)(co * NPQ + pq) * V * rt.lpr;
#pragma unroll
            for (int i = 0; i < V; i++) {
                own[co][pq][i] = s[co][pq][i];
                row[i * rt.lpr + lane] = s[co][pq][i];
            }
        }
    __syncthreads();
}

// Segment variant of stage_source_rows (no ReLU mask): the team owns voxels
// [xs, xs + V * lpr) of row (z, y).  A staged row holds the segment in the usual layout, then
// `dil` values to the left of it and `dil` values to the right (zeros outside the row), which
// the lanes 0 .. 2 dil - 1 load one each.  Ends with a workgroup barrier.
template <int NDIM, int WOUT, int V>
__device__ __forceinline__ void stage_source_segment(const Geom &g, const RowTeams &rt, const RowSegments &sg,
                                                     const View<const float> &gy, int b, int z, int y, int xs,
                                                     int lane, bool rowok, float *__restrict__ S,
                                                     float (&own)[WOUT][RowTaps<NDIM>::NPQ][V],
                                                     const UpperDilations up = UpperDilations{{0, 0}})
{
    constexpr int NZ = Taps<NDIM>::NZ, NPQ = RowTaps<NDIM>::NPQ;
    const int rs = V * rt.lpr + sg.halo;         // floats per staged row (the halo is sized for the larger dilation)
    const bool inrow = rowok && xs + lane * V < g.W;   // lanes past the row stage zeros ...
    const int x0 = min(xs + lane * V, g.W - V);        // ... read from a valid address
    const int h = lane;                          // halo element of this lane, if any
#pragma unroll
    for (int co = 0; co < WOUT; co++) {
        const int dil = dilation_of(g, up, co);
        const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, dil) : single_source();
        const AxisSources sy = adjoint_sources(y, g.H, dil);
        const int hx = h < dil ? xs - dil + h : xs + V * rt.lpr + (h - dil);
        const bool hin = rowok && h < 2 * dil && hx >= 0 && hx < g.W;
        const int hxc = min(max(hx, 0), g.W - 1);
        const bool folds = y < dil || y + dil >= g.H || (NDIM == 3 && (z < dil || z + dil >= g.D));
        const float *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc;
        float s[NPQ][V], sh[NPQ];
        auto add_row = [&](int pq, int cz, int cy, bool ok, bool first) {
            cz = min(max(cz, 0), g.D - 1);
            cy = min(max(cy, 0), g.H - 1);
            const float *rowp = gc + (int64_t)cz * gy.sz + (int64_t)cy * gy.sy;
            float m[V];
            load_vec<V>(rowp + x0, m);
            const float mh = rowp[hxc];
#pragma unroll
            for (int i = 0; i < V; i++) s[pq][i] = (first ? 0.f : s[pq][i]) + (ok && inrow ? m[i] : 0.f);
            sh[pq] = (first ? 0.f : sh[pq]) + (ok && hin ? mh : 0.f);
        };
#pragma unroll
        for (int p = 0; p < NZ; p++)
#pragma unroll
            for (int q = 0; q < 3; q++)
                add_row(p * 3 + q, sz.c[p][0], sy.c[q][0], sz.ok[p][0] && sy.ok[q][0], true);
        if (folds) {
#pragma unroll
            for (int p = 0; p < NZ; p++)
#pragma unroll
                for (int q = 0; q < 3; q++) {
                    add_row(p * 3 + q, sz.c[p][0], sy.c[q][1], sz.ok[p][0] && sy.ok[q][1], false);
                    if (NDIM == 3) {
                        add_row(p * 3 + q, sz.c[p][1], sy.c[q][0], sz.ok[p][1] && sy.ok[q][0], false);
                        add_row(p * 3 + q, sz.c[p][1], sy.c[q][1], sz.ok[p][1] && sy.ok[q][1], false);
                    }
                }
        }
#pragma unroll
        for (int pq = 0; pq < NPQ; pq++) {
            float *row = S + (size_t)(co * NPQ + pq) * rs;
#pragma unroll
            for (int i = 0; i < V; i++) {
                own[co][pq][i] = s[pq][i];
                row[i * rt.lpr + lane] = s[pq][i];
            }
            if (h < 2 * dil) row[V * rt.lpr + h] = sh[pq];
        }
    }
    __syncthreads();
}

// Position of element x in a staged row.
template <int V>
__device__ __forceinline__ int staged_index(int x, int lpr)
{
    return (x % V) * lpr + x / V;
}

// The two x-taps that are not the centre, for voxel x of a staged row:
//   tap 0 (reads x + dil forward):  S[x + dil] if inside,  + S[dil - x - 1]         if x < dil
//   tap 2 (reads x - dil forward):  S[x - dil] if inside,  + S[2W - x - 1 - dil]    if x + dil >= W
// The four LDS positions and masks depend on x only, so they are computed once
// per voxel and reused for every staged row.
template <int V>
struct SideTaps {
    int i0a, i0b, i2a, i2b;
    bool m0a, m0b, m2a, m2b;

    __device__ __forceinline__ SideTaps(int x, int W, int dil, int lpr)
    {
        const int hi = x + dil, lo = x - dil;
        i0a = staged_index<V>(min(hi, W - 1), lpr);
        i0b = staged_index<V>(max(dil - x - 1, 0), lpr);
        i2a = staged_index<V>(max(lo, 0), lpr);
        i2b = staged_index<V>(min(max(2 * W - x - 1 - dil, 0), W - 1), lpr);
        m0a = hi < W;
        m0b = x < dil;
        m2a = lo >= 0;
        m2b = hi >= W;
    }

    // Segment variant: x is a position in the row, the staged row holds [xs, xs + segw) in the
    // usual layout followed by dil values to the left and dil values to the right of it.
    __device__ __forceinline__ SideTaps(int x, int W, int dil, int lpr, int xs, int segw)
    {
        const int hi = x + dil, lo = x - dil;
        auto at = [&](int p) {                   // p: position in the row that this segment stages
            const int j = p - xs;
            return j < 0 ? V * lpr + (j + dil) : (j >= segw ? V * lpr + dil + (j - segw) : staged_index<V>(j, lpr));
        };
        i0a = at(min(hi, W - 1));
        i0b = at(min(max(dil - x - 1, 0), W - 1));
        i2a = at(max(lo, 0));
        i2b = at(min(max(2 * W - x - 1 - dil, 0), W - 1));
        m0a = hi < W;
        m0b = x < dil;
        m2a = lo >= 0;
        m2b = hi >= W;
        // the mirrored sources lie in the first and the last segment only: clamp what the
        // other segments compute for them (masked off) into the staged range
        const int last = V * lpr + 2 * dil - 1;
        i0b = m0b ? i0b : 0;
        i2b = m2b ? i2b : 0;
        i0a = min(max(i0a, 0), last);
        i2a = min(max(i2a, 0), last);
        i0b = min(max(i0b, 0), last);
        i2b = min(max(i2b, 0), last);
    }

    __device__ __forceinline__ void read(const float *__restrict__ row, float &t0, float &t2) const
    {
        const float a0 = row[i0a], b0 = row[i0b], a2 = row[i2a], b2 = row[i2b];
        t0 = (m0a ? a0 : 0.f) + (m0b ? b0 : 0.f);
        t2 = (m2a ? a2 : 0.f) + (m2b ? b2 : 0.f);
    }
};

}  // namespace msd
