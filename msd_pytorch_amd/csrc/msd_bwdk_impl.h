// backward_k (+ bias) for fp32 with unit x-stride, on the matrix cores:
//     grad_kernel[co][ci][t] += sum_u x[ci][u] * A[co][t](u),   grad_bias[co] += sum_u A[co][centre](u)
// with A the adjoint-form gather (msd_adjoint.h) of m = grad_output * [0 < output].
// Per output channel this is a GEMM  D[tap][channel] = A[tap][voxel] * X[voxel][channel]
// whose long dimension (voxels) is the contraction, so it maps onto
// v_mfma_f32_16x16x4_f32 with taps as rows (9 of 16 in 2D, 27 of 2x16 in 3D),
// 16 input channels as columns and 4 voxels per instruction.
//
// Two kernels per call (three with the ReLU mask):
//   mask_gradient   m = grad_output * [0 < output] into a contiguous scratch plane
//                   (skipped for the plain operator, which reads grad_output itself);
//   bwdk_mfma       every WAVE walks its own run of tiles of 64*V consecutive voxels.
//                   Per tile every lane gathers the K taps of its own V voxels straight
//                   from m (coalesced, branch-free loads), a wave-private LDS tile
//                   [tap][voxel] turns them into the MFMA A layout (lane = tap + 16 *
//                   voxel group, registers); then the wave streams the input channels in
//                   blocks of 16: coalesced V-wide loads of its 64*V voxels, a
//                   wave-private LDS tile to turn them into the B layout
//                   (lane = channel + 16 * voxel group), MFMAs, with the next block's loads
//                   issued before the MFMAs of the current one.  No workgroup barrier in
//                   the loop: waves drift freely and hide each other's latencies.  The D
//                   accumulators stay in registers over all tiles; at the end the four
//                   waves of a workgroup are added in LDS and one column-major row of
//                   partial sums per workgroup goes to the workspace;
//   reduce_columns  adds the partial rows in a fixed order and accumulates into
//                   grad_kernel / grad_bias.
// A virtual input channel of ones yields the bias sum.
// Algorithmic traffic: (C + 2w) * N * 4 bytes.
#pragma once
#include "msd_adjoint.h"
#include "msd_kernels.h"
#include "msd_rows.h"

#include <algorithm>

namespace msd {
namespace bwdk {

typedef float mfma4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kChanBlock = 16;

// Wave-private LDS tile: first [tap][voxel] while the A operands are set up,
// then [channel][voxel] in the channel loop.
template <int V> struct XTile {
    static constexpr int kVox = kWave * V;        // voxels per wave tile
    static constexpr int kStride = kVox + 4;      // floats per row (bank spread for the b128 reads)
    static constexpr int kRows = 27;              // >= taps (27 in 3D) and >= kChanBlock
    static constexpr int kFloats = kRows * kStride;
};

// m[b][co][voxel] = grad_output * [0 < output], contiguous.
static __global__ __launch_bounds__(256) void mask_gradient(Geom g, View<const float> out, View<const float> gy,
                                                            float *__restrict__ m)
{
    const int64_t total = (int64_t)g.B * g.Wd * g.nvox;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int n = (int)(i % g.nvox);
        const int64_t bc = i / g.nvox;
        const int co = (int)(bc % g.Wd), b = (int)(bc / g.Wd);
        int z, y, x;
        decode_voxel(g, n, z, y, x);
        const float o = out.p[(int64_t)b * out.sb + (int64_t)co * out.sc + (int64_t)z * out.sz + (int64_t)y * out.sy + x];
        const float v = gy.p[(int64_t)b * gy.sb + (int64_t)co * gy.sc + (int64_t)z * gy.sz + (int64_t)y * gy.sy + x];
        m[i] = 0.f < o ? v : 0.f;
    }
}

template <int NDIM, int V, int NCB>
__global__ __launch_bounds__(kThreads, 2) void bwdk_mfma(Geom g, int remap, int tiles_per_wave, int64_t ntiles,
                                                         int tiles_per_image, View<const float> m,
                                                         View<const float> x, float *__restrict__ part,
                                                         int want_bias)
{
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K;
    constexpr int TG = NDIM == 3 ? 2 : 1;         // groups of 16 tap rows
    constexpr int NS = 4 * V;                     // 16-voxel MFMA groups per wave tile
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), wl = tid % kWave;
    const int mk = wl / 16, mj = wl % 16;         // MFMA k (voxel) and i/j (tap or channel) of this lane
    float *XS = lds + (size_t)wave * XTile<V>::kFloats;

    const int co = blockIdx.z % g.Wd;
    const int chunk = blockIdx.z / g.Wd;
    const int c0 = chunk * NCB * kChanBlock;
    const int ones_ch = want_bias ? g.C : -1;     // virtual channel of ones -> bias sum
    const int c_end = min(g.C + (want_bias ? 1 : 0), c0 + NCB * kChanBlock);
    const int ncb = (c_end - c0 + kChanBlock - 1) / kChanBlock;
    const float inv_w = 1.f / (float)g.W, inv_h = 1.f / (float)g.H;

    mfma4 D[NCB][TG];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++) D[cb][tg] = mfma4{0.f, 0.f, 0.f, 0.f};

    const int lb = block_for_xcd(blockIdx.x, gridDim.x, remap);
    // the four waves of a workgroup take neighbouring tiles, so that together they
    // read 4 * 64 * V consecutive voxels of every channel at about the same time
    const int64_t first = (int64_t)lb * kWaves * tiles_per_wave + wave;

    for (int ti = 0; ti < tiles_per_wave; ti++) {
        const int64_t t = first + (int64_t)ti * kWaves;
        if (t >= ntiles) break;                   // uniform over the wave; no workgroup barrier inside the loop
        int64_t xsc = x.sc;
        asm volatile("" : "+s"(xsc));             // keeps the 16 channel offsets from being hoisted out of the loop
        const int b = (int)(t / tiles_per_image);
        const int n0 = (int)(t % tiles_per_image) * XTile<V>::kVox;
        // position of the first voxel of the tile; everything else is a small offset from it
        const int row0 = n0 / g.W, xb = n0 % g.W;
        const int yb = row0 % g.H, zb = row0 / g.H;
        auto locate = [&](int off, int &z, int &y, int &xx) {
            const int xs = xb + off;                               // < W + 256: the float quotient is exact
            const int q = (int)(((float)xs + 0.5f) * inv_w);
            xx = xs - q * g.W;
            const int ys = yb + q;
            const int qz = (int)(((float)ys + 0.5f) * inv_h);
            y = ys - qz * g.H;
            z = zb + qz;
        };

        // ---- input values of 16 channels for this lane's V voxels (B operand, before the transpose)
        const bool act = n0 + wl * V < g.nvox;
        int lz, ly, lx;
        locate(min(wl * V, g.nvox - V - n0), lz, ly, lx);
        const float *xp0 = x.p + (int64_t)b * x.sb + (int64_t)lz * x.sz + (int64_t)ly * x.sy + lx;
        float xv[kChanBlock][V];
        auto load_block = [&](int cb) {
            // branch-free: clamped channel index, all 16 loads in flight together
#pragma unroll
            for (int c = 0; c < kChanBlock; c++)
                load_vec<V>(xp0 + (int64_t)min(c0 + cb * kChanBlock + c, g.C - 1) * xsc, xv[c]);
        };
        auto fix_block = [&](int cb) {
#pragma unroll
            for (int c = 0; c < kChanBlock; c++) {
                const int ch = c0 + cb * kChanBlock + c;
                const bool keep = act && ch < g.C;
                const float fill = (act && ch == ones_ch) ? 1.f : 0.f;
#pragma unroll
                for (int i = 0; i < V; i++) xv[c][i] = keep ? xv[c][i] : fill;
            }
        };
        load_block(0);   // issued ahead of the gather so the two latencies overlap

        // ---- A operands.  Step 1, voxel layout: every lane gathers the K taps of its own V
        // voxels from m.  Consecutive lanes read consecutive addresses (coalesced); all loads
        // go to clamped, always valid addresses and are masked afterwards, so there is no
        // branch around them and they are all in flight together.
        const float *mc = m.p + (int64_t)b * m.sb + (int64_t)co * m.sc;
        {
            const AxisSources sz = NDIM == 3 ? adjoint_sources(lz, g.D, g.dil) : single_source();
            const AxisSources sy = adjoint_sources(ly, g.H, g.dil);
            // x sources of voxel lx + i: tap 0 reads x + dil (and the fold partner dil - x - 1),
            // tap 2 reads x - dil (and 2W - x - 1 - dil)
            int c0a[V], c0b[V], c2a[V], c2b[V];
            bool k0a[V], k0b[V], k2a[V], k2b[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                const int xx = lx + i;
                c0a[i] = min(xx + g.dil, g.W - 1);                        k0a[i] = xx + g.dil < g.W;
                c0b[i] = max(g.dil - xx - 1, 0);                          k0b[i] = xx < g.dil;
                c2a[i] = max(xx - g.dil, 0);                              k2a[i] = xx >= g.dil;
                c2b[i] = min(max(2 * g.W - xx - 1 - g.dil, 0), g.W - 1);  k2b[i] = xx + g.dil >= g.W;
            }
            float tv[K][V];
            auto add_rows = [&](int a_, int b_, bool first) {
#pragma unroll
                for (int p = 0; p < Taps<NDIM>::NZ; p++)
#pragma unroll
                    for (int q = 0; q < 3; q++) {
                        const int pz = NDIM == 3 ? p : 0;
                        const int cz = min(max(sz.c[pz][a_], 0), g.D - 1), cy = min(max(sy.c[q][b_], 0), g.H - 1);
                        const bool use = act && sz.ok[pz][a_] && sy.ok[q][b_];
                        const float *row = mc + (int64_t)cz * m.sz + (int64_t)cy * m.sy;
                        float mid[V];
                        load_vec<V>(row + lx, mid);
#pragma unroll
                        for (int i = 0; i < V; i++) {
                            const float v0a = row[c0a[i]], v0b = row[c0b[i]], v2a = row[c2a[i]], v2b = row[c2b[i]];
                            const float t0 = (use && k0a[i] ? v0a : 0.f) + (use && k0b[i] ? v0b : 0.f);
                            const float t1 = use ? mid[i] : 0.f;
                            const float t2 = (use && k2a[i] ? v2a : 0.f) + (use && k2b[i] ? v2b : 0.f);
                            const int t = (p * 3 + q) * 3;
                            tv[t + 0][i] = first ? t0 : tv[t + 0][i] + t0;
                            tv[t + 1][i] = first ? t1 : tv[t + 1][i] + t1;
                            tv[t + 2][i] = first ? t2 : tv[t + 2][i] + t2;
                        }
                    }
            };
            add_rows(0, 0, true);
            const bool folds = ly < g.dil || ly + g.dil >= g.H || (NDIM == 3 && (lz < g.dil || lz + g.dil >= g.D));
            if (folds) {   // rows within dil of a y or z border: the fold maps a second row onto some taps
                add_rows(0, 1, false);
                if (NDIM == 3) {
                    add_rows(1, 0, false);
                    add_rows(1, 1, false);
                }
            }
            // Step 2: through a wave-private LDS tile [tap][voxel] into the MFMA layout.
#pragma unroll
            for (int t = 0; t < K; t++) store_vec<V>(XS + t * XTile<V>::kStride + wl * V, tv[t]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // a[tg][s][e] = A[tap = tg*16 + mj](voxel n0 + 16 s + 4 mk + e)
        float a[TG][NS][4];
#pragma unroll
        for (int tg = 0; tg < TG; tg++) {
            const int tap = tg * 16 + mj;
            const float *arow = XS + min(tap, K - 1) * XTile<V>::kStride + 4 * mk;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const f32x4 av = *reinterpret_cast<const f32x4 *>(arow + 16 * s);
#pragma unroll
                for (int e = 0; e < 4; e++) a[tg][s][e] = tap < K ? av[e] : 0.f;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ---- channel loop.  Runtime loop: unrolled, the per-channel addresses and predicates of
        // all NCB blocks would be computed up front and spill.
#pragma unroll 1
        for (int cb = 0; cb < ncb; cb++) {
            fix_block(cb);
#pragma unroll
            for (int c = 0; c < kChanBlock; c++) store_vec<V>(XS + c * XTile<V>::kStride + wl * V, xv[c]);
            // the tile is private to the wave and LDS executes a wave's accesses in
            // order: only the compiler has to be kept from reordering them
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (cb + 1 < ncb) load_block(cb + 1);   // in flight while the matrix cores work on this block
            mfma4 acc[TG][2];                     // two independent accumulation chains per tap group
#pragma unroll
            for (int tg = 0; tg < TG; tg++) acc[tg][0] = acc[tg][1] = mfma4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const f32x4 bv = *reinterpret_cast<const f32x4 *>(XS + mj * XTile<V>::kStride + 16 * s + 4 * mk);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int tg = 0; tg < TG; tg++)
                        acc[tg][e & 1] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(a[tg][s][e], bv[e], acc[tg][e & 1], 0, 0, 0);
            }
            // D is indexed statically: pick the block with a chain of uniform branches
#pragma unroll
            for (int q = 0; q < NCB; q++)
                if (q == cb) {
#pragma unroll
                    for (int tg = 0; tg < TG; tg++) D[q][tg] += acc[tg][0] + acc[tg][1];
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }

    // D[cb][tg][v] = sum for tap tg*16 + 4*mk + v, channel c0 + cb*16 + mj.  Add the four waves in LDS.
    __syncthreads();
    constexpr int PER_WAVE = NCB * TG * 4 * kWave;
    float *red = lds;
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave * PER_WAVE + ((cb * TG + tg) * 4 + v) * kWave + wl] = D[cb][tg][v];
    __syncthreads();
    // partial sums are stored column-major, part[column][workgroup], so that the
    // second pass reads each column as one contiguous run
    float *pcol = part + blockIdx.x;
    for (int idx = tid; idx < PER_WAVE; idx += kThreads) {
        const int l = idx % kWave, v = (idx / kWave) % 4, tg = (idx / (4 * kWave)) % TG, cb = idx / (4 * kWave * TG);
        const int tap = tg * 16 + 4 * (l / 16) + v;
        const int ch = c0 + cb * kChanBlock + l % 16;
        if (tap >= K || ch >= c_end) continue;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) s += red[w * PER_WAVE + idx];
        if (ch < g.C)
            pcol[(((int64_t)co * g.C + ch) * K + tap) * kMaxPartialRows] = s;
        else if (tap == K / 2)
            pcol[((int64_t)g.Wd * g.C * K + co) * kMaxPartialRows] = s;
    }
}

// Second pass: one wave per column of the partial sums.  Lane l adds rows
// l, l + 64, ... in order, then the 64 lane sums are added by a fixed shuffle
// tree, so the result does not depend on scheduling.  Columns [0, nk) go to the
// weight gradient, the following ones to the bias gradient; both accumulate.
static __global__ __launch_bounds__(256) void reduce_columns(const float *__restrict__ part, int rows, int64_t nk,
                                                             int64_t ncols, float *__restrict__ gk,
                                                             float *__restrict__ gb)
{
    const int64_t col = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    if (col >= ncols) return;
    const int l = threadIdx.x % kWave;
    const float *p = part + col * kMaxPartialRows;
    float s = 0.f;
    for (int r = l; r < rows; r += kWave) s += p[r];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_down(s, off, kWave);
    if (l == 0) {
        if (col < nk) {
            gk[col] += s;
        } else {
            gb[col - nk] += s;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Row-team variant.  The gather of the A operands is the one backward_x uses (msd_rows.h): the
// teams of a workgroup stage the source rows of their image rows in LDS once (coalesced V-wide
// loads, the ReLU mask applied on the way in), and every lane takes the K taps of its own V
// voxels from there.  From then on the waves are on their own, as above: LDS transpose into the
// MFMA A layout, then the input channels in blocks of 16.  A workgroup walks `tiles_per_wg`
// groups of rows and keeps its sums in registers until the end.

template <int NDIM, int V> struct RowXTile {
    static constexpr int kVox = kWave * V;
    static constexpr int kStride = kVox + 4;
    static constexpr int kRows = Taps<NDIM>::K > kChanBlock ? Taps<NDIM>::K : kChanBlock;
    static constexpr int kFloats = kRows * kStride;
};

template <int NDIM, bool RELU, int V, int NCB>
__global__ __launch_bounds__(kThreads, 2) void bwdk_rows(Geom g, RowTeams rt, int remap, int tiles_per_wg, int ngroups,
                                                         int total_groups, View<const float> out,
                                                         View<const float> gy, View<const float> x,
                                                         float *__restrict__ part, int want_bias)
{
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K, NPQ = RowTaps<NDIM>::NPQ;
    constexpr int TG = NDIM == 3 ? 2 : 1;         // groups of 16 tap rows
    constexpr int NS = 4 * V;                     // 16-voxel MFMA groups per wave tile
    constexpr int XSTRIDE = RowXTile<NDIM, V>::kStride;
    const int tid = threadIdx.x;
    const int nwaves = blockDim.x / kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), wl = tid % kWave;
    const int mk = wl / 16, mj = wl % 16;         // MFMA k (voxel) and i/j (tap or channel) of this lane
    const int team = tid / rt.lpr, lane = tid % rt.lpr;
    float *S = lds + (size_t)team * NPQ * V * rt.lpr;
    float *XS = lds + (size_t)rt.rpw * NPQ * V * rt.lpr + (size_t)wave * RowXTile<NDIM, V>::kFloats;

    const int co = blockIdx.z % g.Wd;
    const int chunk = blockIdx.z / g.Wd;
    const int c0 = chunk * NCB * kChanBlock;
    const int ones_ch = want_bias ? g.C : -1;     // virtual channel of ones -> bias sum
    const int c_end = min(g.C + (want_bias ? 1 : 0), c0 + NCB * kChanBlock);
    const int ncb = (c_end - c0 + kChanBlock - 1) / kChanBlock;
    // the staging code indexes output channels from 0: shift the views to this one
    View<const float> outc = out, gyc = gy;
    if (RELU) outc.p += (int64_t)co * out.sc;
    gyc.p += (int64_t)co * gy.sc;

    mfma4 D[NCB][TG];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++) D[cb][tg] = mfma4{0.f, 0.f, 0.f, 0.f};

    const int lb = block_for_xcd(blockIdx.x, gridDim.x, remap);
    const int x0 = lane * V;
    const int xc = min(x0, g.W - V);

    for (int ti = 0; ti < tiles_per_wg; ti++) {
        const int grp = lb * tiles_per_wg + ti;
        if (grp >= total_groups) break;           // uniform over the workgroup
        int64_t xsc = x.sc;
        asm volatile("" : "+s"(xsc));             // keeps the 16 channel offsets from being hoisted out of the loop
        const int b = grp / ngroups;
        const int row = (grp % ngroups) * rt.rpw + team;
        const bool act = row < rt.nrows && x0 < g.W;
        const int rr = min(row, rt.nrows - 1);
        const int y = rr % g.H, z = rr / g.H;

        // ---- input values of 16 channels for this lane's V voxels (B operand, before the transpose)
        const float *xp0 = x.p + (int64_t)b * x.sb + (int64_t)z * x.sz + (int64_t)y * x.sy + xc;
        float xv[kChanBlock][V];
        auto load_block = [&](int cb) {
            // branch-free: clamped channel index, all 16 loads in flight together
#pragma unroll
            for (int c = 0; c < kChanBlock; c++)
                load_vec<V>(xp0 + (int64_t)min(c0 + cb * kChanBlock + c, g.C - 1) * xsc, xv[c]);
        };
        auto fix_block = [&](int cb) {
#pragma unroll
            for (int c = 0; c < kChanBlock; c++) {
                const int ch = c0 + cb * kChanBlock + c;
                const bool keep = act && ch < g.C;
                const float fill = (act && ch == ones_ch) ? 1.f : 0.f;
#pragma unroll
                for (int i = 0; i < V; i++) xv[c][i] = keep ? xv[c][i] : fill;
            }
        };
        load_block(0);   // issued ahead of the gather so the two latencies overlap

        // ---- A operands, voxel layout: tv[t][i] = A[t](voxel x0 + i of the team's row)
        {
            float tv[K][V];
            float own[1][NPQ][V];
            stage_source_rows<NDIM, RELU, 1, V>(g, rt, outc, gyc, b, z, y, lane, act, S, own);
#pragma unroll
            for (int i = 0; i < V; i++) {
                const SideTaps<V> side(min(x0 + i, g.W - 1), g.W, g.dil, rt.lpr);
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    side.read(S + (size_t)pq * V * rt.lpr, tv[pq * 3 + 0][i], tv[pq * 3 + 2][i]);
                    tv[pq * 3 + 1][i] = own[0][pq][i];
                }
            }
#pragma unroll
            for (int t = 0; t < K; t++)
#pragma unroll
                for (int i = 0; i < V; i++) tv[t][i] = act ? tv[t][i] : 0.f;
            __syncthreads();                      // the staged rows may be overwritten from here on
            // through a wave-private LDS tile [tap][voxel] into the MFMA layout
#pragma unroll
            for (int t = 0; t < K; t++) store_vec<V>(XS + t * XSTRIDE + wl * V, tv[t]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // a[tg][s][e] = A[tap = tg*16 + mj](wave voxel 16 s + 4 mk + e)
        float a[TG][NS][4];
#pragma unroll
        for (int tg = 0; tg < TG; tg++) {
            const int tap = tg * 16 + mj;
            const float *arow = XS + min(tap, K - 1) * XSTRIDE + 4 * mk;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const f32x4 av = *reinterpret_cast<const f32x4 *>(arow + 16 * s);
#pragma unroll
                for (int e = 0; e < 4; e++) a[tg][s][e] = tap < K ? av[e] : 0.f;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ---- channel loop (runtime loop: unrolled, the addresses of all blocks would be live at once)
#pragma unroll 1
        for (int cb = 0; cb < ncb; cb++) {
            fix_block(cb);
#pragma unroll
            for (int c = 0; c < kChanBlock; c++) store_vec<V>(XS + c * XSTRIDE + wl * V, xv[c]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (cb + 1 < ncb) load_block(cb + 1);   // in flight while the matrix cores work on this block
            mfma4 acc[TG][2];                     // two independent accumulation chains per tap group
#pragma unroll
            for (int tg = 0; tg < TG; tg++) acc[tg][0] = acc[tg][1] = mfma4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const f32x4 bv = *reinterpret_cast<const f32x4 *>(XS + mj * XSTRIDE + 16 * s + 4 * mk);
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int tg = 0; tg < TG; tg++)
                        acc[tg][e & 1] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(a[tg][s][e], bv[e], acc[tg][e & 1], 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < NCB; q++)
                if (q == cb) {
#pragma unroll
                    for (int tg = 0; tg < TG; tg++) D[q][tg] += acc[tg][0] + acc[tg][1];
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }

    // D[cb][tg][v] = sum for tap tg*16 + 4*mk + v, channel c0 + cb*16 + mj.  Add the waves in LDS.
    __syncthreads();
    constexpr int PER_WAVE = NCB * TG * 4 * kWave;
    float *red = lds;
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave * PER_WAVE + ((cb * TG + tg) * 4 + v) * kWave + wl] = D[cb][tg][v];
    __syncthreads();
    float *pcol = part + blockIdx.x;
    for (int idx = tid; idx < PER_WAVE; idx += blockDim.x) {
        const int l = idx % kWave, v = (idx / kWave) % 4, tg = (idx / (4 * kWave)) % TG, cb = idx / (4 * kWave * TG);
        const int tap = tg * 16 + 4 * (l / 16) + v;
        const int ch = c0 + cb * kChanBlock + l % 16;
        if (tap >= K || ch >= c_end) continue;
        float s = 0.f;
        for (int w = 0; w < nwaves; w++) s += red[w * PER_WAVE + idx];
        if (ch < g.C)
            pcol[(((int64_t)co * g.C + ch) * K + tap) * kMaxPartialRows] = s;
        else if (tap == K / 2)
            pcol[((int64_t)g.Wd * g.C * K + co) * kMaxPartialRows] = s;
    }
}

template <int NDIM, int V, int NCB>
size_t rows_lds_bytes(const RowTeams &rt)
{
    constexpr int TG = NDIM == 3 ? 2 : 1;
    const size_t main_loop =
        ((size_t)rt.rpw * RowTaps<NDIM>::NPQ * V * rt.lpr + (size_t)kWaves * RowXTile<NDIM, V>::kFloats) * 4;
    const size_t epilogue = (size_t)kWaves * NCB * TG * 4 * kWave * 4;
    return std::max(main_loop, epilogue);
}

// Row-team kernel usable: rows fit a 256-lane workgroup, V-wide accesses aligned.
template <int NDIM>
bool rows_fit(const Geom &g, bool relu, int V, const View<const float> &out, const View<const float> &gy,
              const View<const float> &x)
{
    RowTeams rt;
    if (!make_row_teams(g, V, &rt) || rt.lpr * rt.rpw > kThreads) return false;
    if (!rows_aligned(x, g.W, V) || !rows_aligned(gy, g.W, V) || (relu && !rows_aligned(out, g.W, V))) return false;
    return g.W >= V;
}

template <int NDIM, bool RELU, int V, int NCB>
hipError_t launch_rows(const Geom &g, const View<const float> &out, const View<const float> &gy,
                       const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    constexpr int K = Taps<NDIM>::K;
    RowTeams rt;
    make_row_teams(g, V, &rt);
    float *part = ws + backward_k_mask_floats(g);
    const int ngroups = (rt.nrows + rt.rpw - 1) / rt.rpw;
    const int64_t total = (int64_t)ngroups * g.B;
    const int remap = knob(kKnobXcdRemap, 1);
    const int64_t max_wgs = std::min<int64_t>(std::max(8, knob(kKnobBwdkBlocks, kMaxPartialRows)), kMaxPartialRows);
    const int tiles_per_wg = (int)((total + max_wgs - 1) / max_wgs);
    const int64_t wgs = (total + tiles_per_wg - 1) / tiles_per_wg;
    const int rows = remap ? xcd_grid((int)wgs) : (int)wgs;   // padding workgroups write zero rows
    if (rows > kMaxPartialRows || total > INT32_MAX) return hipErrorInvalidConfiguration;
    const int want_bias = gb != nullptr;
    const int chunks = (g.C + want_bias + NCB * kChanBlock - 1) / (NCB * kChanBlock);
    const size_t lds = rows_lds_bytes<NDIM, V, NCB>(rt);
    hipLaunchKernelGGL((bwdk_rows<NDIM, RELU, V, NCB>), dim3(rows, 1, chunks * g.Wd), dim3(rt.lpr * rt.rpw), lds, s, g,
                       rt, remap, tiles_per_wg, ngroups, (int)total, out, gy, x, part, want_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nk = (int64_t)g.Wd * g.C * K;
    const int64_t ncols = nk + (want_bias ? g.Wd : 0);
    hipLaunchKernelGGL(reduce_columns, dim3((ncols + 3) / 4), dim3(256), 0, s, part, rows, nk, ncols, gk, gb);
    return hipGetLastError();
}

template <int NDIM, bool RELU, int V>
hipError_t rows_pick_ncb(const Geom &g, const View<const float> &out, const View<const float> &gy,
                         const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    const int need = (g.C + (gb != nullptr) + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch_rows<NDIM, RELU, V, 1>(g, out, gy, x, gk, gb, ws, s);
    if (need <= 2) return launch_rows<NDIM, RELU, V, 2>(g, out, gy, x, gk, gb, ws, s);
    if (need <= 4) return launch_rows<NDIM, RELU, V, 4>(g, out, gy, x, gk, gb, ws, s);
    return launch_rows<NDIM, RELU, V, 8>(g, out, gy, x, gk, gb, ws, s);
}

// Voxels per lane of the row-team kernel: the widest aligned one up to vmax, 0 if none fits.
template <int NDIM>
int rows_choose_vec(const Geom &g, bool relu, int vmax, const View<const float> &out, const View<const float> &gy,
                    const View<const float> &x)
{
    for (int v = NDIM == 3 ? 2 : 4; v >= 1; v /= 2) {
        if (v > vmax) continue;
        if (rows_fit<NDIM>(g, relu, v, out, gy, x)) return v;
    }
    return 0;
}

template <int NDIM, bool RELU>
hipError_t rows_run(const Geom &g, int v, const View<const float> &out, const View<const float> &gy,
                    const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    if constexpr (NDIM == 2) {
        if (v == 4) return rows_pick_ncb<2, RELU, 4>(g, out, gy, x, gk, gb, ws, s);
    }
    if (v == 2) return rows_pick_ncb<NDIM, RELU, 2>(g, out, gy, x, gk, gb, ws, s);
    if (v == 1) return rows_pick_ncb<NDIM, RELU, 1>(g, out, gy, x, gk, gb, ws, s);
    return hipErrorInvalidConfiguration;
}

template <int NDIM, int V, int NCB>
size_t lds_bytes()
{
    constexpr int TG = NDIM == 3 ? 2 : 1;
    const size_t main_loop = (size_t)kWaves * XTile<V>::kFloats * 4;
    const size_t epilogue = (size_t)kWaves * NCB * TG * 4 * kWave * 4;
    return std::max(main_loop, epilogue);
}

template <int NDIM, int V, int NCB>
hipError_t launch(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    constexpr int K = Taps<NDIM>::K;
    View<const float> m = gy;
    float *part = ws;
    if (relu) {
        float *mbuf = ws;
        part = ws + backward_k_mask_floats(g);
        const int64_t total = (int64_t)g.B * g.Wd * g.nvox;
        const int blocks = (int)std::min<int64_t>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(mask_gradient, dim3(blocks), dim3(256), 0, s, g, out, gy, mbuf);
        m = View<const float>{mbuf, (int64_t)g.Wd * g.nvox, (int64_t)g.nvox, (int64_t)g.H * g.W, (int64_t)g.W, 1};
    }
    const int tiles_per_image = (g.nvox + XTile<V>::kVox - 1) / XTile<V>::kVox;
    const int64_t ntiles = (int64_t)tiles_per_image * g.B;
    const int remap = knob(kKnobXcdRemap, 1);
    int64_t wgs = std::min<int64_t>((ntiles + kWaves - 1) / kWaves, knob(kKnobBwdkBlocks, kMaxPartialRows));
    wgs = std::min<int64_t>(wgs, kMaxPartialRows);
    const int tiles_per_wave = (int)((ntiles + wgs * kWaves - 1) / (wgs * kWaves));
    wgs = (ntiles + (int64_t)tiles_per_wave * kWaves - 1) / ((int64_t)tiles_per_wave * kWaves);
    const int rows = remap ? xcd_grid((int)wgs) : (int)wgs;   // padding workgroups write zero rows
    if (rows > kMaxPartialRows) return hipErrorInvalidConfiguration;
    const int want_bias = gb != nullptr;
    const int chunks = (g.C + want_bias + NCB * kChanBlock - 1) / (NCB * kChanBlock);
    const size_t lds = lds_bytes<NDIM, V, NCB>();
    hipLaunchKernelGGL((bwdk_mfma<NDIM, V, NCB>), dim3(rows, 1, chunks * g.Wd), dim3(kThreads), lds, s, g, remap,
                       tiles_per_wave, ntiles, tiles_per_image, m, x, part, want_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nk = (int64_t)g.Wd * g.C * K;
    const int64_t ncols = nk + (want_bias ? g.Wd : 0);
    hipLaunchKernelGGL(reduce_columns, dim3((ncols + 3) / 4), dim3(256), 0, s, part, rows, nk, ncols, gk, gb);
    return hipGetLastError();
}

template <int NDIM, int V>
hipError_t pick_ncb(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                    const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    const int need = (g.C + (gb != nullptr) + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch<NDIM, V, 1>(g, relu, out, gy, x, gk, gb, ws, s);
    if (need <= 2) return launch<NDIM, V, 2>(g, relu, out, gy, x, gk, gb, ws, s);
    if (need <= 4) return launch<NDIM, V, 4>(g, relu, out, gy, x, gk, gb, ws, s);
    return launch<NDIM, V, 8>(g, relu, out, gy, x, gk, gb, ws, s);
}

// Voxels per lane: V-wide accesses to the input must be aligned, and groups of
// four consecutive voxels must not straddle rows (W % 4 == 0).
inline int choose_vec(const Geom &g, int vmax, const View<const float> &x)
{
    if (g.W % 4 != 0 || g.nvox < 4) return 0;
    for (int v = 4; v >= 2; v /= 2) {
        if (v > vmax) continue;
        if (rows_aligned(x, g.W, v)) return v;
    }
    return 0;
}

template <int NDIM>
bool supported_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x)
{
    if (x.sx != 1 || gy.sx != 1 || (relu && out.sx != 1)) return false;
    return rows_choose_vec<NDIM>(g, relu, 4, out, gy, x) != 0 || choose_vec(g, 4, x) != 0;
}

template <int NDIM>
hipError_t run_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    const int vmax = knob(NDIM == 3 ? kKnobBwdkVec3d : kKnobBwdkVec2d, NDIM == 3 ? 2 : 4);
    if (knob(kKnobBwdkRows, 1)) {
        int rv = rows_choose_vec<NDIM>(g, relu, vmax, out, gy, x);
        if (rv == 0) rv = rows_choose_vec<NDIM>(g, relu, 4, out, gy, x);
        if (rv != 0)
            return relu ? rows_run<NDIM, true>(g, rv, out, gy, x, gk, gb, ws, s)
                        : rows_run<NDIM, false>(g, rv, out, gy, x, gk, gb, ws, s);
    }
    int v = choose_vec(g, vmax, x);
    if (v == 0) v = choose_vec(g, 4, x);
    if (v == 4) return pick_ncb<NDIM, 4>(g, relu, out, gy, x, gk, gb, ws, s);
    if (v == 2) return pick_ncb<NDIM, 2>(g, relu, out, gy, x, gk, gb, ws, s);
    return hipErrorInvalidConfiguration;
}

}  // namespace bwdk
}  // namespace msd
