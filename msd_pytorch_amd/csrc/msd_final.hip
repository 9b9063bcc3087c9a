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
#include "msd_rows.h"

#include <algorithm>
#include <initializer_list>
#include <mutex>
#include <utility>
#include <vector>

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

// Final layer, loss and the loss's gradient in one pass over the stack:
//     out = bias + w . x              (NLL: out = log_softmax over the output channels of that)
//     loss = mean of (out - t)^2 | |out - t| | -out[label]
//     g = d loss / d (bias + w . x)   written to gout
// and, for the layer's own parameters, the partial sums of  sum_n g[o][n] * x[c][n]  and
// sum_n g[o][n]  (a second walk over the channels of the same voxels, which the caches
// serve): everything the backward pass needs from the stack, so that it does not have to read
// the stack again.  Columns of `part`: (o, c) -> o * C + c, then c_out bias columns, then the loss.
template <typename T, int V, int MAXO, int KIND>
__global__ __launch_bounds__(kFinalThreads) void final_forward_loss_kernel(
    int64_t nvec, int C, int c_out, const T *__restrict__ x, int64_t xsb, int64_t xsc, const T *__restrict__ w,
    const T *__restrict__ bias, const void *__restrict__ target, int64_t tsb, int64_t tsc, T *__restrict__ out,
    int64_t osb, int64_t osc, T *__restrict__ gout, int64_t gsb, int64_t gsc, T inv_n, int want_sums,
    T *__restrict__ part, int64_t rows)
{
    const int64_t i = (int64_t)blockIdx.x * kFinalThreads + threadIdx.x;
    const bool active = i < nvec;
    const int64_t ic = active ? i : nvec - 1;     // lanes past the end work on a valid voxel and contribute zeros
    const int b = blockIdx.y;
    const int lane = threadIdx.x % kWave;
    const int64_t row = ((int64_t)b * gridDim.x + blockIdx.x) * (kFinalThreads / kWave) + threadIdx.x / kWave;
    const T *xp = x + (int64_t)b * xsb + ic * V;
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
            const T wv = w[(int64_t)min(o, c_out - 1) * C + c];
#pragma unroll
            for (int e = 0; e < V; e++) acc[o][e] += wv * v[e];
        }
    }
    T g[MAXO][V];
    T lsum = T(0);
    if constexpr (KIND == 2) {
        // log-softmax over the output channels, then the negative log-likelihood of the label
        const int64_t *lab = static_cast<const int64_t *>(target) + (int64_t)b * tsb + ic * V;
#pragma unroll
        for (int e = 0; e < V; e++) {
            T m = acc[0][e] + (bias ? bias[0] : T(0));
#pragma unroll
            for (int o = 0; o < MAXO; o++) {
                acc[o][e] += bias && o < c_out ? bias[o] : T(0);
                if (o < c_out) m = acc[o][e] > m ? acc[o][e] : m;
            }
            T se = T(0);
#pragma unroll
            for (int o = 0; o < MAXO; o++)
                if (o < c_out) se += exp(acc[o][e] - m);
            const T lse = m + log(se);
            const int64_t t = lab[e];
#pragma unroll
            for (int o = 0; o < MAXO; o++) {
                acc[o][e] -= lse;                             // log-probability
                const T pr = o < c_out ? exp(acc[o][e]) : T(0);
                g[o][e] = active && o < c_out ? (pr - (t == o ? T(1) : T(0))) * inv_n : T(0);
                if (active && t == o) lsum -= acc[o][e];
            }
        }
    } else {
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            const bool keep = active && o < c_out;
            T t[V];
            load_elems<T, V>(static_cast<const T *>(target) + (int64_t)b * tsb + (int64_t)min(o, c_out - 1) * tsc + ic * V,
                             t);
            const T bv = bias && o < c_out ? bias[o] : T(0);
#pragma unroll
            for (int e = 0; e < V; e++) {
                acc[o][e] += bv;
                const T diff = acc[o][e] - t[e];
                if (KIND == 0) {
                    g[o][e] = keep ? T(2) * diff * inv_n : T(0);
                    lsum += keep ? diff * diff : T(0);
                } else {
                    g[o][e] = keep ? (diff > T(0) ? inv_n : (diff < T(0) ? -inv_n : T(0))) : T(0);
                    lsum += keep ? (diff < T(0) ? -diff : diff) : T(0);
                }
            }
        }
    }
    if (active) {
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            if (o >= c_out) break;
            store_elems<T, V>(out + (int64_t)b * osb + (int64_t)o * osc + i * V, acc[o]);
            store_elems<T, V>(gout + (int64_t)b * gsb + (int64_t)o * gsc + i * V, g[o]);
        }
    }
    lsum = wave_sum(lsum * inv_n);
    if (lane == 0) part[((int64_t)c_out * C + c_out) * rows + row] = lsum;
    if (!want_sums) return;                                   // uniform
#pragma unroll
    for (int o = 0; o < MAXO; o++) {
        T sb = T(0);
#pragma unroll
        for (int e = 0; e < V; e++) sb += g[o][e];
        sb = wave_sum(sb);
        if (lane == 0 && o < c_out) part[((int64_t)c_out * C + o) * rows + row] = sb;
    }
    // (from the last channel to the first: what the first walk read last is still in the caches)
#pragma unroll 2
    for (int c = C - 1; c >= 0; c--) {
        T v[V];
        load_elems<T, V>(xp + (int64_t)c * xsc, v);
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            T sw = T(0);
#pragma unroll
            for (int e = 0; e < V; e++) sw += g[o][e] * v[e];
            sw = wave_sum(sw);
            if (lane == 0 && o < c_out) part[((int64_t)o * C + c) * rows + row] = sw;
        }
    }
}

// The same pass for up to 128 input channels with the stack read ONCE (fp32): a workgroup of
// eight waves owns a tile of 64 * V voxels; lane l of every wave stands for the same V voxels
// and wave w takes the channels c % 8 == w.  First walk: each wave loads its channels of the
// tile (all requests issued before the first use), adds its share of the outputs and leaves
// the values in LDS; the eight partial outputs meet in LDS, every wave forms the loss
// gradient g of its lanes' voxels; second walk: each wave takes its channels back from LDS
// and adds g * x to per-lane running sums, which live in registers over all tiles of the
// workgroup (tile t, t + grid, ...) and are reduced over the lanes once at the end: one row
// of partial sums per workgroup.  Same columns of `part` as the kernel above.
constexpr int kTiledWaves = 8;
constexpr int kTiledThreads = kTiledWaves * kWave;
constexpr int kTiledMaxChannels = 128;

template <int V, int MAXO, int KIND, int CC>
__global__ __launch_bounds__(kTiledThreads, 4) void final_forward_loss_tiled(
    int64_t nvec, int tiles_per_image, int total_tiles, int C, int c_out, const float *__restrict__ x, int64_t xsb,
    int64_t xsc, const float *__restrict__ w, const float *__restrict__ bias, const void *__restrict__ target,
    int64_t tsb, int64_t tsc, float *__restrict__ out, int64_t osb, int64_t osc, float *__restrict__ gout, int64_t gsb,
    int64_t gsc, float inv_n, int want_sums, float *__restrict__ part, int64_t rows)
{
    extern __shared__ float lds_tile[];
    // weights and bias are read-only for the whole kernel: addressed as constant memory they
    // are wave-uniform scalar loads (as plain global loads next to the stores of the loop they
    // would each take a vector register)
    typedef const __attribute__((address_space(4))) float *const_floats_t;
    const const_floats_t wk = (const_floats_t)(uintptr_t)w;
    const const_floats_t bk = (const_floats_t)(uintptr_t)bias;
    constexpr int TV = kWave * V;                             // voxels of a tile
    float *red = lds_tile + (size_t)C * TV;                   // [wave][o][e][lane]; then g as [o][e][lane]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
    float sw[MAXO][CC], sb[MAXO], lsum = 0.f;
#pragma unroll
    for (int o = 0; o < MAXO; o++) {
        sb[o] = 0.f;
#pragma unroll
        for (int cc = 0; cc < CC; cc++) sw[o][cc] = 0.f;
    }
    // this wave's weights: w[o][c] for c = cc * 8 + wave (zero past the last channel)
    for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
        // new values as far as the compiler knows: the weights (scalar loads) and the channels'
        // offsets are formed again per tile instead of being kept, and spilled, over the loop
        asm volatile("" : "+s"(xsc), "+s"(C));
        const int b = tile / tiles_per_image;
        const int64_t i = (int64_t)(tile - b * tiles_per_image) * kWave + lane;
        const bool active = i < nvec;
        const int64_t ic = active ? i : nvec - 1;             // lanes past the end work on a valid voxel, contribute zeros
        // a uniform base per channel plus one 32-bit lane offset: no address registers per request
        const uint64_t xbase = reinterpret_cast<uint64_t>(x + (int64_t)b * xsb);
        const uint32_t xoff = (uint32_t)(ic * V) * 4u;
        float acc[MAXO][V];
#pragma unroll
        for (int o = 0; o < MAXO; o++)
#pragma unroll
            for (int e = 0; e < V; e++) acc[o][e] = 0.f;
        // channels in groups of G requests, all of a group issued before its first use: all of
        // the wave's channels at once where the running sums leave the registers for it
        constexpr int G = MAXO * CC + V * CC < 96 ? CC : (CC < 24 / V ? CC : 24 / V);
#pragma unroll
        for (int c0 = 0; c0 < CC; c0 += G) {
            float v[G][V];
#pragma unroll
            for (int j = 0; j < G; j++)
                load_global_vec<V>(xbase + (uint64_t)((int64_t)min((c0 + j) * kTiledWaves + wave, C - 1) * xsc * 4), xoff,
                                   v[j]);
#pragma unroll
            for (int j = 0; j < G; j++) {
                const int c = (c0 + j) * kTiledWaves + wave;  // uniform
                if (c < C) {
#pragma unroll
                    for (int o = 0; o < MAXO; o++) {
                        const float wv = wk[(int64_t)min(o, c_out - 1) * C + c];
#pragma unroll
                        for (int e = 0; e < V; e++) acc[o][e] += wv * v[j][e];
                    }
                    store_elems<float, V>(lds_tile + (size_t)c * TV + lane * V, v[j]);
                }
            }
        }
#pragma unroll
        for (int o = 0; o < MAXO; o++)
#pragma unroll
            for (int e = 0; e < V; e++) red[((wave * MAXO + o) * V + e) * kWave + lane] = acc[o][e];
        __syncthreads();
        // the eight partial outputs in a fixed order (a loop that stays a loop: unrolled, all
        // 8 * MAXO * V values would be requested at once and held in registers)
#pragma unroll
        for (int o = 0; o < MAXO; o++)
#pragma unroll
            for (int e = 0; e < V; e++) acc[o][e] = red[(o * V + e) * kWave + lane];
#pragma unroll 1
        for (int q = 1; q < kTiledWaves; q++) {
            const float *rq = red + (size_t)q * MAXO * V * kWave + lane;
#pragma unroll
            for (int o = 0; o < MAXO; o++)
#pragma unroll
                for (int e = 0; e < V; e++) acc[o][e] += rq[(o * V + e) * kWave];
        }
        float g[MAXO][V];
        float tile_loss = 0.f;
        if constexpr (KIND == 2) {
            // the softmax is the expensive part: wave q forms it for element q of every lane's
            // voxels only, and the waves exchange the results through LDS below
            const int64_t *lab = static_cast<const int64_t *>(target) + (int64_t)b * tsb + ic * V;
#pragma unroll
            for (int e = 0; e < V; e++) {
                if (wave != e) continue;                      // uniform
                float m = acc[0][e] + (bias ? bk[0] : 0.f);
#pragma unroll
                for (int o = 0; o < MAXO; o++) {
                    acc[o][e] += bias && o < c_out ? bk[o] : 0.f;
                    if (o < c_out) m = acc[o][e] > m ? acc[o][e] : m;
                }
                float se = 0.f;
#pragma unroll
                for (int o = 0; o < MAXO; o++)
                    if (o < c_out) se += exp(acc[o][e] - m);
                const float lse = m + log(se);
                const int64_t t = lab[e];
#pragma unroll
                for (int o = 0; o < MAXO; o++) {
                    acc[o][e] -= lse;                         // log-probability
                    const float pr = o < c_out ? exp(acc[o][e]) : 0.f;
                    g[o][e] = active && o < c_out ? (pr - (t == o ? 1.f : 0.f)) * inv_n : 0.f;
                    if (active && t == o) tile_loss -= acc[o][e];
                }
            }
        } else {
#pragma unroll
            for (int o = 0; o < MAXO; o++) {
                const bool keep = active && o < c_out;
                float t[V];
                load_elems<float, V>(static_cast<const float *>(target) + (int64_t)b * tsb +
                                         (int64_t)min(o, c_out - 1) * tsc + ic * V, t);
                const float bv = bias && o < c_out ? bk[o] : 0.f;
#pragma unroll
                for (int e = 0; e < V; e++) {
                    acc[o][e] += bv;
                    const float diff = acc[o][e] - t[e];
                    if (KIND == 0) {
                        g[o][e] = keep ? 2.f * diff * inv_n : 0.f;
                        tile_loss += keep ? diff * diff : 0.f;
                    } else {
                        g[o][e] = keep ? (diff > 0.f ? inv_n : (diff < 0.f ? -inv_n : 0.f)) : 0.f;
                        tile_loss += keep ? (diff < 0.f ? -diff : diff) : 0.f;
                    }
                }
            }
        }
        if constexpr (KIND == 2) {
            // wave e wrote nothing of the other elements: log-probabilities and g through LDS
            __syncthreads();                                  // all waves have read the partial outputs
            float *gs = red, *ls = red + MAXO * V * kWave;    // [o][e][lane] each
#pragma unroll
            for (int e = 0; e < V; e++)
                if (wave == e) {
#pragma unroll
                    for (int o = 0; o < MAXO; o++) {
                        gs[(o * V + e) * kWave + lane] = g[o][e];
                        ls[(o * V + e) * kWave + lane] = acc[o][e];
                    }
                }
            __syncthreads();
#pragma unroll
            for (int o = 0; o < MAXO; o++)
#pragma unroll
                for (int e = 0; e < V; e++) {
                    g[o][e] = gs[(o * V + e) * kWave + lane];
                    acc[o][e] = ls[(o * V + e) * kWave + lane];
                }
            // (tile_loss: each of the waves 0 .. V - 1 holds the terms of its element)
        }
        if (wave == 0 || (KIND == 2 && wave < V)) lsum += tile_loss * inv_n;
        if (wave == 0) {                                      // uniform: one wave writes the outputs
            if (active) {
#pragma unroll
                for (int o = 0; o < MAXO; o++) {
                    if (o >= c_out) break;
                    store_elems<float, V>(out + (int64_t)b * osb + (int64_t)o * osc + i * V, acc[o]);
                    store_elems<float, V>(gout + (int64_t)b * gsb + (int64_t)o * gsc + i * V, g[o]);
                }
            }
#pragma unroll
            for (int o = 0; o < MAXO; o++)
#pragma unroll
                for (int e = 0; e < V; e++) sb[o] += g[o][e];
        }
        if (want_sums) {                                      // uniform
#pragma unroll
            for (int cc = 0; cc < CC; cc++) {
                const int c = cc * kTiledWaves + wave;
                if (c < C) {
                    float xv[V];
                    load_elems<float, V>(lds_tile + (size_t)c * TV + lane * V, xv);   // what this wave stored itself
#pragma unroll
                    for (int o = 0; o < MAXO; o++)
#pragma unroll
                        for (int e = 0; e < V; e++) sw[o][cc] += g[o][e] * xv[e];
                }
            }
        }
        __syncthreads();                                      // `red` is rewritten by the next tile
    }
    const int64_t row = blockIdx.x;
    {
        // the loss terms of the waves that hold some (wave 0; NLL: waves 0 .. V - 1), in order
        lsum = wave_sum(lsum);
        if (lane == 0) red[wave] = lsum;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = red[0];
            if constexpr (KIND == 2)
                for (int q = 1; q < V; q++) t += red[q];
            part[((int64_t)c_out * C + c_out) * rows + row] = t;
        }
    }
    if (!want_sums) return;
    if (wave == 0) {
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            const float s = wave_sum(sb[o]);
            if (lane == 0 && o < c_out) part[((int64_t)c_out * C + o) * rows + row] = s;
        }
    }
#pragma unroll
    for (int cc = 0; cc < CC; cc++) {
        const int c = cc * kTiledWaves + wave;
#pragma unroll
        for (int o = 0; o < MAXO; o++) {
            const float s = wave_sum(sw[o][cc]);
            if (lane == 0 && o < c_out && c < C) part[((int64_t)o * C + c) * rows + row] = s;
        }
    }
}

// One workgroup per column: thread t adds rows t, t + 256, ... in order, a fixed shuffle tree
// adds the lanes of each wave and the four wave sums are added in order.
// Columns [0, nw) go to gw, [nw, nw + nb) to gb, a last one (if any) to `loss`.
template <typename T>
__global__ __launch_bounds__(256) void final_reduce_kernel(const T *__restrict__ part, int64_t rows, int64_t nw,
                                                           int64_t nb, T *__restrict__ gw, T *__restrict__ gb,
                                                           T *__restrict__ loss)
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
        } else if (col < nw + nb) {
            if (gb) gb[col - nw] = total;
        } else if (loss) {
            *loss = total;
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
    return (c_out * c_in + c_out + 1) * final_rows(batch, nvox);   // weight, bias and loss columns
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
    hipLaunchKernelGGL(final_reduce_kernel<T>, dim3((unsigned)ncols), dim3(256), 0, s, ws, rows, nw, (int64_t)c_out, gw,
                       gb, (T *)nullptr);
    return hipGetLastError();
}

namespace {

// Kernels that ask for more than 64 KB of LDS need the attribute set once per kernel and
// device (it stays); later launches, also ones recorded into a graph, go without the call.
hipError_t allow_large_lds(const void *kernel, size_t bytes)
{
    static std::mutex mutex;
    static std::vector<std::pair<const void *, int>> done;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mutex);
    for (const auto &d : done)
        if (d.first == kernel && d.second == dev) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) done.emplace_back(kernel, dev);
    return e;
}

constexpr size_t kTiledLdsLimit = 80 * 1024;     // two workgroups share the 160 KB of a CU

template <int V, int MAXO, int KIND, int CC>
hipError_t launch_tiled(int64_t batch, int c_in, int c_out, int64_t nvox, const float *x, int64_t xsb, int64_t xsc,
                        const float *w, const float *bias, const void *target, int64_t tsb, int64_t tsc, float *out,
                        int64_t osb, int64_t osc, float *gout, int64_t gsb, int64_t gsc, float inv_n, int want,
                        float *ws, int64_t *rows, hipStream_t s)
{
    const int64_t nvec = nvox / V;
    const int64_t tiles_per_image = (nvec + kWave - 1) / kWave;
    const int64_t total = tiles_per_image * batch;
    if (total > INT32_MAX) return hipErrorInvalidConfiguration;
    const size_t lds = ((size_t)c_in * kWave * V + (size_t)kTiledWaves * MAXO * V * kWave) * sizeof(float);
    const void *fn = reinterpret_cast<const void *>(&final_forward_loss_tiled<V, MAXO, KIND, CC>);
    if (lds > 64 * 1024) {
        const hipError_t e = allow_large_lds(fn, kTiledLdsLimit);
        if (e != hipSuccess) return e;
    }
    const int grid = (int)std::min<int64_t>(total, 512);      // two workgroups per CU, each walks its tiles
    *rows = grid;
    hipLaunchKernelGGL((final_forward_loss_tiled<V, MAXO, KIND, CC>), dim3(grid), dim3(kTiledThreads), lds, s, nvec,
                       (int)tiles_per_image, (int)total, c_in, c_out, x, xsb, xsc, w, bias, target, tsb, tsc, out, osb,
                       osc, gout, gsb, gsc, inv_n, want, ws, (int64_t)grid);
    return hipGetLastError();
}

// V-wide accesses at multiples of V are aligned in every view given.
inline bool vec_aligned(int v, int64_t nvox, std::initializer_list<std::pair<const void *, std::pair<int64_t, int64_t>>> views)
{
    if (nvox % v != 0) return false;
    for (const auto &vw : views) {
        if (!vw.first) continue;
        if (reinterpret_cast<uintptr_t>(vw.first) % (v * sizeof(float)) != 0 || vw.second.first % v != 0 ||
            vw.second.second % v != 0)
            return false;
    }
    return true;
}

// The tiled kernel where it applies (fp32, up to 128 input and 4 output channels, a tile that
// fits the LDS); *handled says whether it was launched.
hipError_t final_forward_loss_tiled_try(int kind, int64_t batch, int c_in, int c_out, int64_t nvox, const float *x,
                                        int64_t xsb, int64_t xsc, const float *w, const float *bias,
                                        const void *target, int64_t tsb, int64_t tsc, float *out, int64_t osb,
                                        int64_t osc, float *gout, int64_t gsb, int64_t gsc, float inv_n, int want,
                                        float *ws, int64_t *rows, hipStream_t s, bool *handled)
{
    *handled = false;
    if (c_in > kTiledMaxChannels || c_out > 4 || !knob(kKnobFinalTiled, 1)) return hipSuccess;
    const int mo = c_out > 2 ? 4 : (c_out > 1 ? 2 : 1);
    int v = 0;
    for (int cand = 4; cand >= 1; cand /= 2) {
        const bool aligned =
            kind == 2 ? vec_aligned(cand, nvox, {{x, {xsb, xsc}}, {out, {osb, osc}}, {gout, {gsb, gsc}}})
                      : vec_aligned(cand, nvox, {{x, {xsb, xsc}}, {out, {osb, osc}}, {gout, {gsb, gsc}}, {target, {tsb, tsc}}});
        const size_t lds = ((size_t)c_in * kWave * cand + (size_t)kTiledWaves * mo * cand * kWave) * sizeof(float);
        if (aligned && lds <= kTiledLdsLimit && (cand < 4 || c_in <= 64)) {
            v = cand;
            break;
        }
    }
    if (v == 0) return hipSuccess;
    const bool wide = c_in > 64;                              // sixteen channels per wave instead of eight
#define MSD_TILED(VV, OO, KK, CCC)                                                                                    \
    return (*handled = true, launch_tiled<VV, OO, KK, CCC>(batch, c_in, c_out, nvox, x, xsb, xsc, w, bias, target, tsb, \
                                                          tsc, out, osb, osc, gout, gsb, gsc, inv_n, want, ws, rows, s))
#define MSD_TILED_C(VV, OO, KK)                                  \
    do {                                                         \
        if (VV == 4 || !wide) MSD_TILED(VV, OO, KK, 8);          \
        if constexpr (VV != 4) MSD_TILED(VV, OO, KK, 16);        \
    } while (0)
#define MSD_TILED_K(VV, OO)                                                                     \
    do {                                                                                        \
        if (kind == 0) MSD_TILED_C(VV, OO, 0); else if (kind == 1) MSD_TILED_C(VV, OO, 1); else MSD_TILED_C(VV, OO, 2); \
    } while (0)
#define MSD_TILED_O(VV)                                                                         \
    do {                                                                                        \
        if (mo == 4) MSD_TILED_K(VV, 4); else if (mo == 2) MSD_TILED_K(VV, 2); else MSD_TILED_K(VV, 1); \
    } while (0)
    if (v == 4) MSD_TILED_O(4); else if (v == 2) MSD_TILED_O(2); else MSD_TILED_O(1);
#undef MSD_TILED_O
#undef MSD_TILED_K
#undef MSD_TILED_C
#undef MSD_TILED
    return hipSuccess;
}

template <typename T> struct TiledLoss {
    static hipError_t run(int, int64_t, int, int, int64_t, const T *, int64_t, int64_t, const T *, const T *,
                          const void *, int64_t, int64_t, T *, int64_t, int64_t, T *, int64_t, int64_t, T, int, T *,
                          int64_t *, hipStream_t, bool *handled)
    {
        *handled = false;
        return hipSuccess;
    }
};
template <> struct TiledLoss<float> {
    template <typename... A> static hipError_t run(A... a) { return final_forward_loss_tiled_try(a...); }
};

}  // namespace

template <typename T>
hipError_t final_forward_loss(int kind, int64_t batch, int c_in, int c_out, int64_t nvox, const T *x, int64_t xsb,
                              int64_t xsc, const T *w, const T *bias, const void *target, int64_t tsb, int64_t tsc,
                              T *out, int64_t osb, int64_t osc, T *gout, int64_t gsb, int64_t gsc, T *gw, T *gb,
                              T *loss, T *ws, hipStream_t s)
{
    {
        const int64_t terms = kind == 2 ? batch * nvox : batch * nvox * (int64_t)c_out;
        bool handled = false;
        int64_t rows = 0;
        const hipError_t e = TiledLoss<T>::run(kind, batch, c_in, c_out, nvox, x, xsb, xsc, w, bias, target, tsb, tsc, out,
                                               osb, osc, gout, gsb, gsc, T(1) / T(terms), (int)(gw || gb), ws, &rows, s,
                                               &handled);
        if (e != hipSuccess) return e;
        if (handled) {
            const int64_t nw = (int64_t)c_out * c_in;
            if (gw || gb) {
                hipLaunchKernelGGL(final_reduce_kernel<T>, dim3((unsigned)(nw + c_out + 1)), dim3(256), 0, s, ws, rows,
                                   nw, (int64_t)c_out, gw, gb, loss);
            } else {
                hipLaunchKernelGGL(final_reduce_kernel<T>, dim3(1), dim3(256), 0, s, ws + (nw + c_out) * rows, rows,
                                   (int64_t)0, (int64_t)0, (T *)nullptr, (T *)nullptr, loss);
            }
            return hipGetLastError();
        }
    }
    // labels are one int64 per voxel: no vector width to match
    const int V = kind == 2 ? final_vec<T>(nvox, {{x, {xsb, xsc}}, {out, {osb, osc}}, {gout, {gsb, gsc}}})
                            : final_vec<T>(nvox, {{x, {xsb, xsc}}, {out, {osb, osc}}, {gout, {gsb, gsc}},
                                                  {target, {tsb, tsc}}});
    const int64_t nvec = nvox / V;
    const dim3 grid((unsigned)((nvec + kFinalThreads - 1) / kFinalThreads), (unsigned)batch, 1);
    const int64_t rows = (int64_t)grid.x * batch * (kFinalThreads / kWave);
    const int64_t terms = kind == 2 ? batch * nvox : batch * nvox * (int64_t)c_out;
    const T inv_n = T(1) / T(terms);
    const int want = gw || gb;
    const int mo = c_out > 4 ? 8 : (c_out > 2 ? 4 : (c_out > 1 ? 2 : 1));
#define MSD_FINAL_LOSS(VV, OO, KK)                                                                                  \
    hipLaunchKernelGGL((final_forward_loss_kernel<T, VV, OO, KK>), grid, dim3(kFinalThreads), 0, s, nvec, c_in, c_out, \
                       x, xsb, xsc, w, bias, target, tsb, tsc, out, osb, osc, gout, gsb, gsc, inv_n, want, ws, rows)
#define MSD_FINAL_LOSS_O(VV, KK)                                                                        \
    do {                                                                                                \
        if (mo == 8) MSD_FINAL_LOSS(VV, 8, KK); else if (mo == 4) MSD_FINAL_LOSS(VV, 4, KK);            \
        else if (mo == 2) MSD_FINAL_LOSS(VV, 2, KK); else MSD_FINAL_LOSS(VV, 1, KK);                    \
    } while (0)
#define MSD_FINAL_LOSS_K(VV)                                                                            \
    do {                                                                                                \
        if (kind == 0) MSD_FINAL_LOSS_O(VV, 0); else if (kind == 1) MSD_FINAL_LOSS_O(VV, 1); else MSD_FINAL_LOSS_O(VV, 2); \
    } while (0)
    if (V == 1) {
        MSD_FINAL_LOSS_K(1);
    } else {
        constexpr int W = wide_vec<T>();
        MSD_FINAL_LOSS_K(W);
    }
#undef MSD_FINAL_LOSS_K
#undef MSD_FINAL_LOSS_O
#undef MSD_FINAL_LOSS
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nw = (int64_t)c_out * c_in;
    if (want) {
        hipLaunchKernelGGL(final_reduce_kernel<T>, dim3((unsigned)(nw + c_out + 1)), dim3(256), 0, s, ws, rows, nw,
                           (int64_t)c_out, gw, gb, loss);
    } else {
        // only the loss column was written
        hipLaunchKernelGGL(final_reduce_kernel<T>, dim3(1), dim3(256), 0, s, ws + (nw + c_out) * rows, rows, (int64_t)0,
                           (int64_t)0, (T *)nullptr, (T *)nullptr, loss);
    }
    return hipGetLastError();
}

template hipError_t final_forward_loss<float>(int, int64_t, int, int, int64_t, const float *, int64_t, int64_t,
                                              const float *, const float *, const void *, int64_t, int64_t, float *,
                                              int64_t, int64_t, float *, int64_t, int64_t, float *, float *, float *,
                                              float *, hipStream_t);
template hipError_t final_forward_loss<double>(int, int64_t, int, int, int64_t, const double *, int64_t, int64_t,
                                               const double *, const double *, const void *, int64_t, int64_t,
                                               double *, int64_t, int64_t, double *, int64_t, int64_t, double *,
                                               double *, double *, double *, hipStream_t);

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
