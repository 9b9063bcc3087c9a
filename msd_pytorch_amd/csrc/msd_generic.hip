// Shape-generic kernels: any strides, any number of output channels, float or
// double.  One lane per voxel.  These carry the double-precision path and every
// fp32 problem that the specialised kernels do not accept.
#include "msd_kernels.h"
#include "msd_adjoint.h"

namespace msd {

namespace {

constexpr int kBlock = 256;



// ---------------------------------------------------------------------------
// Forward: out = [max(0, .)] (bias + sum_ci sum_taps x[fold(v + dil*tap)] * k)
// Accumulation order per output: bias first, channels outer, taps row-major.
// COT output channels share each loaded input value.
// ---------------------------------------------------------------------------
template <typename T, int NDIM, bool RELU, int COT>
__global__ __launch_bounds__(kBlock) void fwd_generic(Geom g, View<const T> x, const T *__restrict__ k,
                                                      const T *__restrict__ bias, View<T> out)
{
    constexpr int NZ = Taps<NDIM>::NZ, K = Taps<NDIM>::K;
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= g.nvox) return;
    const int b = blockIdx.y;
    const int co0 = blockIdx.z * COT;
    int z, y, xx;
    decode_voxel(g, n, z, y, xx);

    int64_t oz[NZ], oy[3], ox[3];
#pragma unroll
    for (int t = 0; t < 3; t++) {
        oy[t] = (int64_t)reflect_idx(y + (t - 1) * g.dil, g.H) * x.sy;
        ox[t] = (int64_t)reflect_idx(xx + (t - 1) * g.dil, g.W) * x.sx;
    }
#pragma unroll
    for (int t = 0; t < NZ; t++)
        oz[t] = NDIM == 3 ? (int64_t)reflect_idx(z + (t - 1) * g.dil, g.D) * x.sz : 0;

    T acc[COT];
    int co[COT];
#pragma unroll
    for (int j = 0; j < COT; j++) {
        co[j] = min(co0 + j, g.Wd - 1);
        acc[j] = bias[co[j]];
    }
    const T *xb = x.p + (int64_t)b * x.sb;
    for (int ci = 0; ci < g.C; ci++) {
        const T *xc = xb + (int64_t)ci * x.sc;
#pragma unroll
        for (int p = 0; p < NZ; p++)
#pragma unroll
            for (int q = 0; q < 3; q++)
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    const T v = xc[oz[p] + oy[q] + ox[r]];
#pragma unroll
                    for (int j = 0; j < COT; j++)
                        acc[j] += v * k[((int64_t)co[j] * g.C + ci) * K + (p * 3 + q) * 3 + r];
                }
    }
    const int64_t o = (int64_t)b * out.sb + (int64_t)z * out.sz + (int64_t)y * out.sy + (int64_t)xx * out.sx;
#pragma unroll
    for (int j = 0; j < COT; j++)
        if (co0 + j < g.Wd) {
            T v = acc[j];
            if (RELU) v = v > T(0) ? v : T(0);
            out.p[o + (int64_t)(co0 + j) * out.sc] = v;
        }
}

// grad_input[b, c0 .. c0+cch) += adjoint; one read-modify-write per output channel.
template <typename T, int NDIM, bool RELU>
__global__ __launch_bounds__(kBlock) void bwdx_generic(Geom g, int cch, View<const T> out, View<const T> gy,
                                                       const T *__restrict__ k, View<T> gx)
{
    constexpr int K = Taps<NDIM>::K;
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= g.nvox) return;
    const int b = blockIdx.y;
    const int c0 = blockIdx.z * cch;
    const int c1 = min(c0 + cch, g.C);
    int z, y, x;
    decode_voxel(g, n, z, y, x);
    T *gxp = gx.p + (int64_t)b * gx.sb + (int64_t)z * gx.sz + (int64_t)y * gx.sy + (int64_t)x * gx.sx;

    for (int co = 0; co < g.Wd; co++) {
        T A[K];
        const T *oc = RELU ? out.p + (int64_t)b * out.sb + (int64_t)co * out.sc : nullptr;
        const T *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc;
        gather_adjoint<T, NDIM, RELU>(g, oc, out, gc, gy, z, y, x, A);
        for (int ci = c0; ci < c1; ci++) {
            const T *kc = k + ((int64_t)co * g.C + ci) * K;
            T s = T(0);
#pragma unroll
            for (int t = 0; t < K; t++) s += kc[t] * A[t];
            gxp[(int64_t)ci * gx.sc] += s;
        }
    }
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    return v;  // valid in lane 0
}

// Sum `v` over the workgroup in a fixed order; the total is returned to thread 0.
template <typename T>
__device__ __forceinline__ T block_sum(T v, T *lds)
{
    v = wave_sum(v);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (threadIdx.x % kWave == 0) lds[wave] = v;
    __syncthreads();
    T s = T(0);
    if (threadIdx.x == 0)
        for (int i = 0; i < kBlock / kWave; i++) s += lds[i];
    return s;
}

// Partial weight (and bias) gradients.  Every workgroup walks a fixed set of
// voxel tiles and keeps private sums for CCH input channels; the sums are
// reduced across the workgroup once and written to
//     part[blockIdx.x][(co * C + ci) * K + t]        (weights)
//     part[blockIdx.x][Wd * C * K + co]              (bias, by blockIdx.y == 0)
// A second kernel adds the partials up in index order, so the result does not
// depend on scheduling.  Voxel index n runs over batch * D * H * W.
template <typename T, int NDIM, bool RELU, int CCH>
__global__ __launch_bounds__(kBlock) void bwdk_generic_partial(Geom g, View<const T> out, View<const T> gy,
                                                               View<const T> x, T *__restrict__ part,
                                                               int want_k, int want_bias)
{
    constexpr int K = Taps<NDIM>::K;
    __shared__ T lds[kBlock / kWave];
    const int c0 = blockIdx.y * CCH;
    const int co = blockIdx.z;
    const int64_t total = (int64_t)g.B * g.nvox;
    const int64_t nout = (int64_t)g.Wd * g.C * K + g.Wd;

    T acc[CCH][K];
    T accb = T(0);
#pragma unroll
    for (int j = 0; j < CCH; j++)
#pragma unroll
        for (int t = 0; t < K; t++) acc[j][t] = T(0);

    for (int64_t n = (int64_t)blockIdx.x * kBlock + threadIdx.x; n < total; n += (int64_t)gridDim.x * kBlock) {
        const int b = (int)(n / g.nvox);
        int z, y, xx;
        decode_voxel(g, (int)(n % g.nvox), z, y, xx);
        T A[K];
        const T *oc = RELU ? out.p + (int64_t)b * out.sb + (int64_t)co * out.sc : nullptr;
        const T *gc = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc;
        gather_adjoint<T, NDIM, RELU>(g, oc, out, gc, gy, z, y, xx, A);
        accb += A[K / 2];
        if (want_k) {
            const T *xp = x.p + (int64_t)b * x.sb + (int64_t)z * x.sz + (int64_t)y * x.sy + (int64_t)xx * x.sx;
#pragma unroll
            for (int j = 0; j < CCH; j++) {
                const int ci = min(c0 + j, g.C - 1);
                const T v = xp[(int64_t)ci * x.sc];
#pragma unroll
                for (int t = 0; t < K; t++) acc[j][t] += v * A[t];
            }
        }
    }

    T *row = part + (int64_t)blockIdx.x * nout;
    if (want_k) {
#pragma unroll
        for (int j = 0; j < CCH; j++)
#pragma unroll
            for (int t = 0; t < K; t++) {
                const T s = block_sum(acc[j][t], lds);
                if (threadIdx.x == 0 && c0 + j < g.C) row[((int64_t)co * g.C + c0 + j) * K + t] = s;
            }
    }
    if (want_bias && blockIdx.y == 0) {
        const T s = block_sum(accb, lds);
        if (threadIdx.x == 0) row[(int64_t)g.Wd * g.C * K + co] = s;
    }
}

// dst[i] += sum over rows of part[row][first + i], rows in increasing order.
template <typename T>
__global__ __launch_bounds__(kBlock) void reduce_partials(const T *__restrict__ part, int rows, int64_t nout,
                                                          int64_t first, int64_t count, T *__restrict__ dst)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= count) return;
    T s = T(0);
    for (int r = 0; r < rows; r++) s += part[(int64_t)r * nout + first + i];
    dst[i] += s;
}

// gy = gy * [0 < out], in place, over batch * Wd * nvox elements.
template <typename T>
__global__ __launch_bounds__(kBlock) void relu_mask_inplace(Geom g, View<const T> out, View<T> gy)
{
    const int64_t total = (int64_t)g.B * g.Wd * g.nvox;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int n = (int)(i % g.nvox);
        const int64_t bc = i / g.nvox;
        const int co = (int)(bc % g.Wd), b = (int)(bc / g.Wd);
        int z, y, x;
        decode_voxel(g, n, z, y, x);
        const T o = out.p[(int64_t)b * out.sb + (int64_t)co * out.sc + (int64_t)z * out.sz + (int64_t)y * out.sy +
                          (int64_t)x * out.sx];
        T *p = gy.p + (int64_t)b * gy.sb + (int64_t)co * gy.sc + (int64_t)z * gy.sz + (int64_t)y * gy.sy +
               (int64_t)x * gy.sx;
        if (!(T(0) < o)) *p = T(0);
    }
}

inline int partial_rows(const Geom &g)
{
    const int64_t total = (int64_t)g.B * g.nvox;
    int64_t rows = (total + kBlock - 1) / kBlock;
    if (rows > kMaxPartialRows) rows = kMaxPartialRows;
    return (int)rows;
}

template <typename T, int NDIM, bool RELU>
hipError_t launch_fwd(const Geom &g, View<const T> x, const T *k, const T *bias, View<T> out, hipStream_t s)
{
    const unsigned gx = (g.nvox + kBlock - 1) / kBlock;
    if (g.Wd == 1) {
        hipLaunchKernelGGL((fwd_generic<T, NDIM, RELU, 1>), dim3(gx, g.B, 1), dim3(kBlock), 0, s, g, x, k, bias, out);
    } else if (g.Wd == 2) {
        hipLaunchKernelGGL((fwd_generic<T, NDIM, RELU, 2>), dim3(gx, g.B, 1), dim3(kBlock), 0, s, g, x, k, bias, out);
    } else {
        hipLaunchKernelGGL((fwd_generic<T, NDIM, RELU, 4>), dim3(gx, g.B, (g.Wd + 3) / 4), dim3(kBlock), 0, s, g, x, k,
                           bias, out);
    }
    return hipGetLastError();
}

template <typename T, int NDIM, bool RELU>
hipError_t launch_bwdx(const Geom &g, View<const T> out, View<const T> gy, const T *k, View<T> gx, hipStream_t s)
{
    const unsigned nb = (g.nvox + kBlock - 1) / kBlock;
    // split the channels over the grid only as far as needed to fill the chip
    int cch = g.C;
    while (cch > 8 && (int64_t)nb * g.B * ((g.C + cch - 1) / cch) < 2048) cch = (cch + 1) / 2;
    hipLaunchKernelGGL((bwdx_generic<T, NDIM, RELU>), dim3(nb, g.B, (g.C + cch - 1) / cch), dim3(kBlock), 0, s, g, cch,
                       out, gy, k, gx);
    return hipGetLastError();
}

template <typename T, int NDIM, bool RELU>
hipError_t launch_bwdk(const Geom &g, View<const T> out, View<const T> gy, View<const T> x, T *gk, T *gb, T *ws,
                       hipStream_t s)
{
    constexpr int K = Taps<NDIM>::K;
    constexpr int CCH = NDIM == 3 ? 2 : 4;
    const int rows = partial_rows(g);
    const int64_t nout = (int64_t)g.Wd * g.C * K + g.Wd;
    const int want_k = gk != nullptr, want_bias = gb != nullptr;
    const int chunks = want_k ? (g.C + CCH - 1) / CCH : 1;
    hipLaunchKernelGGL((bwdk_generic_partial<T, NDIM, RELU, CCH>), dim3(rows, chunks, g.Wd), dim3(kBlock), 0, s, g, out,
                       gy, x, ws, want_k, want_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (want_k) {
        const int64_t cnt = (int64_t)g.Wd * g.C * K;
        hipLaunchKernelGGL((reduce_partials<T>), dim3((cnt + kBlock - 1) / kBlock), dim3(kBlock), 0, s, ws, rows, nout,
                           (int64_t)0, cnt, gk);
    }
    if (want_bias) {
        hipLaunchKernelGGL((reduce_partials<T>), dim3(1), dim3(kBlock), 0, s, ws, rows, nout,
                           (int64_t)g.Wd * g.C * K, (int64_t)g.Wd, gb);
    }
    return hipGetLastError();
}

}  // namespace

int64_t generic_workspace_elems(const Geom &g)
{
    const int K = g.ndim == 3 ? 27 : 9;
    // sized for the largest row count any backward_k path uses
    return backward_k_mask_floats(g) + (int64_t)kMaxPartialRows * ((int64_t)g.Wd * g.C * K + g.Wd);
}

template <typename T>
hipError_t generic_forward(const Geom &g, bool relu, View<const T> x, const T *k, const T *bias, View<T> out,
                           hipStream_t s)
{
    if (g.ndim == 2)
        return relu ? launch_fwd<T, 2, true>(g, x, k, bias, out, s) : launch_fwd<T, 2, false>(g, x, k, bias, out, s);
    return relu ? launch_fwd<T, 3, true>(g, x, k, bias, out, s) : launch_fwd<T, 3, false>(g, x, k, bias, out, s);
}

template <typename T>
hipError_t generic_backward_x(const Geom &g, bool relu, View<const T> out, View<const T> gy, const T *k, View<T> gx,
                              hipStream_t s)
{
    if (g.ndim == 2)
        return relu ? launch_bwdx<T, 2, true>(g, out, gy, k, gx, s) : launch_bwdx<T, 2, false>(g, out, gy, k, gx, s);
    return relu ? launch_bwdx<T, 3, true>(g, out, gy, k, gx, s) : launch_bwdx<T, 3, false>(g, out, gy, k, gx, s);
}

template <typename T>
hipError_t generic_backward_kb(const Geom &g, bool relu, View<const T> out, View<const T> gy, View<const T> x, T *gk,
                               T *gb, T *ws, hipStream_t s)
{
    if (g.ndim == 2)
        return relu ? launch_bwdk<T, 2, true>(g, out, gy, x, gk, gb, ws, s)
                    : launch_bwdk<T, 2, false>(g, out, gy, x, gk, gb, ws, s);
    return relu ? launch_bwdk<T, 3, true>(g, out, gy, x, gk, gb, ws, s)
                : launch_bwdk<T, 3, false>(g, out, gy, x, gk, gb, ws, s);
}

template <typename T>
hipError_t generic_relu_mask(const Geom &g, View<const T> out, View<T> gy, hipStream_t s)
{
    const int64_t total = (int64_t)g.B * g.Wd * g.nvox;
    const int blocks = (int)((total + kBlock - 1) / kBlock < 8192 ? (total + kBlock - 1) / kBlock : 8192);
    hipLaunchKernelGGL((relu_mask_inplace<T>), dim3(blocks), dim3(kBlock), 0, s, g, out, gy);
    return hipGetLastError();
}

#define MSD_INSTANTIATE(T)                                                                                         \
    template hipError_t generic_forward<T>(const Geom &, bool, View<const T>, const T *, const T *, View<T>,       \
                                           hipStream_t);                                                           \
    template hipError_t generic_backward_x<T>(const Geom &, bool, View<const T>, View<const T>, const T *, View<T>, \
                                              hipStream_t);                                                        \
    template hipError_t generic_relu_mask<T>(const Geom &, View<const T>, View<T>, hipStream_t);                     \
    template hipError_t generic_backward_kb<T>(const Geom &, bool, View<const T>, View<const T>, View<const T>,    \
                                               T *, T *, T *, hipStream_t);
MSD_INSTANTIATE(float)
MSD_INSTANTIATE(double)

}  // namespace msd
