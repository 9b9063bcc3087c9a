// Device helpers shared by the backward kernels: tap counts, voxel decoding and
// the adjoint-form gather of the (masked) output gradient.
#pragma once

#include "msd_common.h"

namespace msd {

template <int NDIM> struct Taps { static constexpr int NZ = NDIM == 3 ? 3 : 1; static constexpr int K = NZ * 9; };

__device__ __forceinline__ void decode_voxel(const Geom &g, int n, int &z, int &y, int &x)
{
    x = n % g.W;
    const int t = n / g.W;
    y = t % g.H;
    z = t / g.H;
}

// ---------------------------------------------------------------------------
// Masked output gradient gathered in adjoint form.  For input voxel u and
// weight tap t, A[t] = sum of m[v] over all output voxels v whose tap t reads
// u, with m = grad_output (* [0 < output] when RELU).  Then
//     grad_input[ci][u]  += sum_t k[co][ci][t] * A[t]            (backward_x)
//     grad_kernel[co][ci][t] = sum_u x[ci][u] * A[t](u)           (backward_k)
//     grad_bias[co]          = sum_u A[centre](u)                 (bias)
// ---------------------------------------------------------------------------
template <typename T, int NDIM, bool RELU>
__device__ __forceinline__ void gather_adjoint(const Geom &g, const T *__restrict__ oc, const View<const T> &ov,
                                               const T *__restrict__ gc, const View<const T> &gv,
                                               int z, int y, int x, T (&A)[Taps<NDIM>::K])
{
    constexpr int NZ = Taps<NDIM>::NZ;
    const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, g.dil) : single_source();
    const AxisSources sy = adjoint_sources(y, g.H, g.dil);
    const AxisSources sx = adjoint_sources(x, g.W, g.dil);
#pragma unroll
    for (int p = 0; p < NZ; p++)
#pragma unroll
        for (int q = 0; q < 3; q++)
#pragma unroll
            for (int r = 0; r < 3; r++) {
                T s = T(0);
#pragma unroll
                for (int a = 0; a < 2; a++) {
                    if (!sz.ok[p][a]) continue;
#pragma unroll
                    for (int bq = 0; bq < 2; bq++) {
                        if (!sy.ok[q][bq]) continue;
#pragma unroll
                        for (int cr = 0; cr < 2; cr++) {
                            if (!sx.ok[r][cr]) continue;
                            const int cz = sz.c[p][a], cy = sy.c[q][bq], cx = sx.c[r][cr];
                            T m = gc[(int64_t)cz * gv.sz + (int64_t)cy * gv.sy + (int64_t)cx * gv.sx];
                            if (RELU) {
                                const T o = oc[(int64_t)cz * ov.sz + (int64_t)cy * ov.sy + (int64_t)cx * ov.sx];
                                m = T(0) < o ? m : T(0);
                            }
                            s += m;
                        }
                    }
                }
                A[(p * 3 + q) * 3 + r] = s;
            }
}

typedef float f32x2u __attribute__((ext_vector_type(2), aligned(4)));
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));

// V consecutive floats from a 4-byte aligned address (one global_load_dwordxV).
template <int V> __device__ __forceinline__ void load_run(const float *p, float (&d)[V]);
template <> __device__ __forceinline__ void load_run<1>(const float *p, float (&d)[1]) { d[0] = *p; }
template <> __device__ __forceinline__ void load_run<2>(const float *p, float (&d)[2])
{
    const f32x2u v = *reinterpret_cast<const f32x2u *>(p);
    d[0] = v[0]; d[1] = v[1];
}
template <> __device__ __forceinline__ void load_run<4>(const float *p, float (&d)[4])
{
    const f32x4u v = *reinterpret_cast<const f32x4u *>(p);
    d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
}

// gather_adjoint for V consecutive voxels x0 .. x0+V-1 of one row (fp32, unit
// x-stride): A[t][i] belongs to voxel x0 + i.  Away from the x borders every
// tap is one run of V consecutive source values, fetched with a single load;
// lanes that touch a border fall back to element-wise gathering for that tap.
template <int NDIM, bool RELU, int V>
__device__ __forceinline__ void gather_adjoint_run(const Geom &g, const float *__restrict__ oc,
                                                   const View<const float> &ov, const float *__restrict__ gc,
                                                   const View<const float> &gv, int z, int y, int x0,
                                                   float (&A)[Taps<NDIM>::K][V])
{
    constexpr int NZ = Taps<NDIM>::NZ;
    const AxisSources sz = NDIM == 3 ? adjoint_sources(z, g.D, g.dil) : single_source();
    const AxisSources sy = adjoint_sources(y, g.H, g.dil);
    // all V voxels at least dil away from both x borders: every tap then has
    // exactly one source per voxel and the sources form a run
    const bool inner = x0 >= g.dil && x0 + V - 1 + g.dil < g.W;
#pragma unroll
    for (int p = 0; p < NZ; p++)
#pragma unroll
        for (int q = 0; q < 3; q++) {
            float acc[3][V];
#pragma unroll
            for (int r = 0; r < 3; r++)
#pragma unroll
                for (int i = 0; i < V; i++) acc[r][i] = 0.f;
#pragma unroll
            for (int a = 0; a < 2; a++) {
                if (!sz.ok[p][a]) continue;
#pragma unroll
                for (int bq = 0; bq < 2; bq++) {
                    if (!sy.ok[q][bq]) continue;
                    const float *grow = gc + (int64_t)sz.c[p][a] * gv.sz + (int64_t)sy.c[q][bq] * gv.sy;
                    const float *orow = RELU ? oc + (int64_t)sz.c[p][a] * ov.sz + (int64_t)sy.c[q][bq] * ov.sy : nullptr;
#pragma unroll
                    for (int r = 0; r < 3; r++) {
                        // tap r reads x + (r-1)*dil in the forward pass, so the
                        // primary source of voxel x is x - (r-1)*dil
                        const int xs = x0 - (r - 1) * g.dil;
                        const bool whole = r == 1 || inner;
                        if (whole) {
                            float m[V];
                            load_run<V>(grow + xs, m);
                            if (RELU) {
                                float o[V];
                                load_run<V>(orow + xs, o);
#pragma unroll
                                for (int i = 0; i < V; i++) m[i] = 0.f < o[i] ? m[i] : 0.f;
                            }
#pragma unroll
                            for (int i = 0; i < V; i++) acc[r][i] += m[i];
                        } else {
#pragma unroll
                            for (int i = 0; i < V; i++) {
                                const AxisSources sx = adjoint_sources(x0 + i, g.W, g.dil);
#pragma unroll
                                for (int cr = 0; cr < 2; cr++) {
                                    if (!sx.ok[r][cr]) continue;
                                    float m = grow[sx.c[r][cr]];
                                    if (RELU) m = 0.f < orow[sx.c[r][cr]] ? m : 0.f;
                                    acc[r][i] += m;
                                }
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 3; r++)
#pragma unroll
                for (int i = 0; i < V; i++) A[(p * 3 + q) * 3 + r][i] = acc[r][i];
        }
}

}  // namespace msd
