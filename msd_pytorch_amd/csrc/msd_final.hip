// Final layer of the network: a 1x1 convolution over the whole channel stack,
//     out[b][o][n] = bias[o] + sum_c w[o][c] * x[b][c][n]
// (the Conv1d over flattened voxels of msd_module.py:60-88), forward and backward, as
// single passes over the stack.  Every thread owns V consecutive voxels and walks the
// channels; the weights are wave-uniform (scalar loads).
//   forward   reads the stack once: (C + c_out) * N elements of traffic;
//   backward  reads the stack once and writes its gradient once, both in the same walk:
//             grad_x[c] = sum_o w[o][c] * g[o]   and   grad_w[o][c] = sum_n g[o][n] * x[c][n].
//             The sums over voxels are reduced per wave with lane shuffles, stored as one
//             row of partial sums per wave and added in a fixed order by a second kernel,
//             so the result does not depend on scheduling.
// Output channels are handled in groups of at most MAXO per launch.
#include "msd_kernels.h"

#include <initializer_list>
#include <utility>

namespace msd {

namespace {

template <typename T, int V> struct VecOf { typedef T type __attribute__((ext_vector_type(V))); };

template <typename T, int V>
__device__ __forceinline__ void load_elems(const T *p, T (&d)[V])
{
    if constexpr (V == 1) {
        d[0] = *p;
    } else {
        const typename VecOf<T, V>::type v = *reinterpret_cast<const typename VecOf<T, V>::type *>(p);
#pragma unroll
        for (int i = 0; i < V; i++) d[i] = v[i];
    }
}

template <typename T, int V>
__device__ __forceinline__ void store_elems(T *p, const T (&d)[V])
{
    if constexpr (V == 1) {
        *p = d[0];
    } else {
        typename VecOf<T, V>::type v;
#pragma unroll
        for (int i = 0; i < V; i++) v[i] = d[i];
        *reinterpret_cast<typename VecOf<T, V>::type *>(p) = v;
    }
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

constexpr int kFinalThreads = 256;

template <typename T, int V, int MAXO>
__global__ __launch_bounds__(kFinalThreads) void final_forward_kernel(int64_t nvec, int C, int c_out, int o0,
                                                                     const T *__restrict__ x, int64_t xsb,
                                                                     int64_t xsc, const T *__restrict__ w,
                                                                     const T *__restrict__ bias, T *__restrict__ out,
                                                                     int64_t osb, int64_t osc)
{
    const int64_t i = (int64_t)blockIdx.x * kFinalThreads + threadIdx.x;
    if (i >= nvec) return;
    const int b = blockIdx.y;
    const T *xp = x + (int64_t)b * xsb + i * V;
    T acc[MAXO][V];
#pragma unroll
    for (int o = 0; o < MAXO; o++)
#pragma unroll
        for (int e = 0; e < V; e++) acc[o][e] = T(0);
#pragma unroll 4
    for (int c = 0; c < C; c++) {
        T v[V];
        load_elems<T, V>(xp + (int64_t)c * xsc, v);
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            const T wv = w[(int64_t)min(o0 + o, c_out - 1) * C + c];   // clamped: the extra sums are dropped
#pragma unroll
            for (int e = 0; e < V; e++) acc[o][e] += wv * v[e];
        }
    }
#pragma unroll
    for (int o = 0; o < MAXO; o++) {
        if (o0 + o >= c_out) break;
        const T bv = bias ? bias[o0 + o] : T(0);
#pragma unroll
        for (int e = 0; e < V; e++) acc[o][e] += bv;
        store_elems<T, V>(out + (int64_t)b * osb + (int64_t)(o0 + o) * osc + i * V, acc[o]);
    }
}

// part[column][row]: one row per wave; columns (o, c) -> o * C + c, then c_out bias columns.
template <typename T, int V, int MAXO>
__global__ __launch_bounds__(kFinalThreads) void final_backward_kernel(int64_t nvec, int C, int c_out, int o0,
                                                                      const T *__restrict__ x, int64_t xsb,
                                                                      int64_t xsc, const T *__restrict__ go,
                                                                      int64_t gsb, int64_t gsc,
                                                                      const T *__restrict__ w, T *__restrict__ gx,
                                                                      int64_t gxsb, int64_t gxsc,
                                                                      T *__restrict__ part, int64_t rows)
{
    const int64_t i = (int64_t)blockIdx.x * kFinalThreads + threadIdx.x;
    const bool active = i < nvec;
    const int64_t ic = active ? i : nvec - 1;     // lanes past the end read a valid address and contribute zeros
    const int b = blockIdx.y;
    const int lane = threadIdx.x % kWave;
    const int64_t row = ((int64_t)b * gridDim.x + blockIdx.x) * (kFinalThreads / kWave) + threadIdx.x / kWave;
    T g[MAXO][V];
#pragma unroll
    for (int o = 0; o < MAXO; o++) {
        load_elems<T, V>(go + (int64_t)b * gsb + (int64_t)min(o0 + o, c_out - 1) * gsc + ic * V, g[o]);
        const bool keep = active && o0 + o < c_out;
#pragma unroll
        for (int e = 0; e < V; e++) g[o][e] = keep ? g[o][e] : T(0);
    }
    // part == nullptr: neither the weight nor the bias gradient is wanted (a frozen layer);
    // the input is then not read at all and only grad_input is written
    const bool want_sums = part != nullptr;       // uniform
    // bias gradient: sum of the output gradient over voxels
    if (want_sums) {
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            T s = T(0);
#pragma unroll
            for (int e = 0; e < V; e++) s += g[o][e];
            s = wave_sum(s);
            if (lane == 0 && o0 + o < c_out) part[((int64_t)c_out * C + o0 + o) * rows + row] = s;
        }
    }
    const T *xp = x + (int64_t)b * xsb + ic * V;
    T *gp = gx ? gx + (int64_t)b * gxsb + ic * V : nullptr;
#pragma unroll 2
    for (int c = 0; c < C; c++) {
        T v[V];
        if (want_sums) load_elems<T, V>(xp + (int64_t)c * xsc, v);
        if (gp) {
            T r[V];
            if (o0 > 0) {                         // later groups of output channels add to the first one's result
                load_elems<T, V>(gp + (int64_t)c * gxsc, r);
            } else {
#pragma unroll
                for (int e = 0; e < V; e++) r[e] = T(0);
            }
#pragma unroll
            for (int o = 0; o < MAXO; o++) {
                const T wv = w[(int64_t)min(o0 + o, c_out - 1) * C + c];   // g is zero for the clamped ones
#pragma unroll
                for (int e = 0; e < V; e++) r[e] += wv * g[o][e];
            }
            if (active) store_elems<T, V>(gp + (int64_t)c * gxsc, r);
        }
        if (want_sums) {
#pragma unroll
            for (int o = 0; o < MAXO; o++) {
                T s = T(0);
#pragma unroll
                for (int e = 0; e < V; e++) s += g[o][e] * v[e];
                s = wave_sum(s);
                if (lane == 0 && o0 + o < c_out) part[((int64_t)(o0 + o) * C + c) * rows + row] = s;
            }
        }
    }
}

// One workgroup per column: thread t adds rows t, t + 256, ... in order, a fixed shuffle tree
// adds the lanes of each wave and the four wave sums are added in order.
template <typename T>
__global__ __launch_bounds__(256) void final_reduce_kernel(const T *__restrict__ part, int64_t rows, int64_t nw,
                                                           int64_t ncols, T *__restrict__ gw, T *__restrict__ gb)
{
    __shared__ T wave_sum[256 / kWave];
    const int64_t col = blockIdx.x;
    const T *p = part + col * rows;
    T s = T(0);
    for (int64_t r = threadIdx.x; r < rows; r += 256) s += p[r];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_down(s, off, kWave);
    if (threadIdx.x % kWave == 0) wave_sum[threadIdx.x / kWave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        T total = wave_sum[0];
        for (int w = 1; w < 256 / kWave; w++) total += wave_sum[w];
        if (col < nw) {
            if (gw) gw[col] = total;
        } else if (gb) {
            gb[col - nw] = total;
        }
    }
}

template <typename T> constexpr int wide_vec() { return 16 / sizeof(T); }

// Widest vector width whose accesses are aligned in every view given.
template <typename T>
int final_vec(int64_t nvox, std::initializer_list<std::pair<const void *, std::pair<int64_t, int64_t>>> views)
{
    const int v = wide_vec<T>();
    if (nvox % v != 0) return 1;
    for (const auto &vw : views) {
        if (!vw.first) continue;
        if (reinterpret_cast<uintptr_t>(vw.first) % 16 != 0 || vw.second.first % v != 0 || vw.second.second % v != 0)
            return 1;
    }
    return v;
}

inline int group_width(int left) { return left >= 8 ? 8 : left >= 4 ? 4 : left >= 2 ? 2 : 1; }

}  // namespace

int64_t final_rows(int64_t batch, int64_t nvox)
{
    // one row per wave of the narrowest launch (V = 1)
    return batch * ((nvox + kFinalThreads - 1) / kFinalThreads) * (kFinalThreads / kWave);
}

int64_t final_workspace_elems(int64_t batch, int64_t c_in, int64_t c_out, int64_t nvox)
{
    return (c_out * c_in + c_out) * final_rows(batch, nvox);
}

template <typename T>
hipError_t final_forward(int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb, int64_t xsc,
                         const T *w, const T *bias, T *out, int64_t osb, int64_t osc, hipStream_t s)
{
    const int V = final_vec<T>(nvox, {{x, {xsb, xsc}}, {out, {osb, osc}}});
    const int64_t nvec = nvox / V;
    const dim3 grid((unsigned)((nvec + kFinalThreads - 1) / kFinalThreads), (unsigned)batch, 1);
    for (int o0 = 0; o0 < c_out;) {
        const int gw = group_width(c_out - o0);
#define MSD_FINAL_FWD(VV, OO)                                                                                       \
    hipLaunchKernelGGL((final_forward_kernel<T, VV, OO>), grid, dim3(kFinalThreads), 0, s, nvec, c_in, c_out, o0, x, \
                       xsb, xsc, w, bias, out, osb, osc)
        if (V == 1) {
            if (gw == 8) MSD_FINAL_FWD(1, 8); else if (gw == 4) MSD_FINAL_FWD(1, 4); else if (gw == 2) MSD_FINAL_FWD(1, 2); else MSD_FINAL_FWD(1, 1);
        } else {
            constexpr int W = wide_vec<T>();
            if (gw == 8) MSD_FINAL_FWD(W, 8); else if (gw == 4) MSD_FINAL_FWD(W, 4); else if (gw == 2) MSD_FINAL_FWD(W, 2); else MSD_FINAL_FWD(W, 1);
        }
#undef MSD_FINAL_FWD
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        o0 += gw;
    }
    return hipSuccess;
}

template <typename T>
hipError_t final_backward(int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb, int64_t xsc,
                          const T *go, int64_t gsb, int64_t gsc, const T *w, T *gx, int64_t gxsb, int64_t gxsc,
                          T *gw, T *gb, T *ws, hipStream_t s)
{
    const int V = final_vec<T>(nvox, {{x, {xsb, xsc}}, {go, {gsb, gsc}}, {gx, {gxsb, gxsc}}});
    const int64_t nvec = nvox / V;
    const dim3 grid((unsigned)((nvec + kFinalThreads - 1) / kFinalThreads), (unsigned)batch, 1);
    const int64_t rows = (int64_t)grid.x * batch * (kFinalThreads / kWave);
    if (!gw && !gb) ws = nullptr;                 // no sums over voxels wanted: no partial sums, no second pass
    if (!ws && !gx) return hipSuccess;
    for (int o0 = 0; o0 < c_out;) {
        const int gwd = group_width(c_out - o0);
#define MSD_FINAL_BWD(VV, OO)                                                                                        \
    hipLaunchKernelGGL((final_backward_kernel<T, VV, OO>), grid, dim3(kFinalThreads), 0, s, nvec, c_in, c_out, o0, x, \
                       xsb, xsc, go, gsb, gsc, w, gx, gxsb, gxsc, ws, rows)
        if (V == 1) {
            if (gwd == 8) MSD_FINAL_BWD(1, 8); else if (gwd == 4) MSD_FINAL_BWD(1, 4); else if (gwd == 2) MSD_FINAL_BWD(1, 2); else MSD_FINAL_BWD(1, 1);
        } else {
            constexpr int W = wide_vec<T>();
            if (gwd == 8) MSD_FINAL_BWD(W, 8); else if (gwd == 4) MSD_FINAL_BWD(W, 4); else if (gwd == 2) MSD_FINAL_BWD(W, 2); else MSD_FINAL_BWD(W, 1);
        }
#undef MSD_FINAL_BWD
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        o0 += gwd;
    }
    if (!ws) return hipSuccess;
    const int64_t nw = (int64_t)c_out * c_in, ncols = nw + c_out;
    hipLaunchKernelGGL(final_reduce_kernel<T>, dim3((unsigned)ncols), dim3(256), 0, s, ws, rows, nw, ncols, gw, gb);
    return hipGetLastError();
}

template hipError_t final_forward<float>(int64_t, int, int, int64_t, const float *, int64_t, int64_t, const float *,
                                         const float *, float *, int64_t, int64_t, hipStream_t);
template hipError_t final_forward<double>(int64_t, int, int, int64_t, const double *, int64_t, int64_t, const double *,
                                          const double *, double *, int64_t, int64_t, hipStream_t);
template hipError_t final_backward<float>(int64_t, int, int, int64_t, const float *, int64_t, int64_t, const float *,
                                          int64_t, int64_t, const float *, float *, int64_t, int64_t, float *, float *,
                                          float *, hipStream_t);
template hipError_t final_backward<double>(int64_t, int, int, int64_t, const double *, int64_t, int64_t,
                                           const double *, int64_t, int64_t, const double *, double *, int64_t, int64_t,
                                           double *, double *, double *, hipStream_t);

}  // namespace msd
