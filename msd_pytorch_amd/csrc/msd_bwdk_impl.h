// backward_k (+ bias) for fp32 with contiguous rows, on the matrix cores:
//     grad_kernel[co][ci][t] += sum_u x[ci][u] * A[co][t](u),   grad_bias[co] += sum_u A[co][centre](u)
// with A the adjoint-form gather of the masked output gradient (msd_rows.h).
// Per output channel this is a GEMM  D[tap][channel] = A[tap][voxel] * X[voxel][channel]
// whose long dimension (voxels) is the contraction, so it maps onto
// v_mfma_f32_16x16x4_f32 with taps as rows (9 of 16 in 2D, 27 of 2x16 in 3D),
// 16 input channels as columns and 4 voxels per instruction.
//
// A workgroup of four waves walks over tiles of 256*V voxels (rows of the
// image, row-team mapping).  Per tile it stages the folded source rows in LDS,
// lets every lane compute the K taps of its own V voxels (as backward_x does),
// passes them through an LDS tile [tap][voxel] into the MFMA A layout
// (registers, lane = tap + 16 * voxel) and then streams the input channels in
// blocks of 16: each wave loads its own
// 64*V voxels of the 16 channels with coalesced V-wide loads, transposes them
// through a wave-private LDS tile into the B layout (lane = channel + 16 * voxel)
// and issues the MFMAs.  The D accumulators stay in registers across all tiles
// of the workgroup; at the end the four waves are added in LDS and one row of
// partial sums per workgroup goes to the workspace, which reduce_partials adds
// up in a fixed order.  A virtual input channel of ones yields the bias sum.
// Algorithmic traffic: (C + 2w) * N * 4 bytes.
#pragma once
#include "msd_kernels.h"
#include "msd_rows.h"

#include <algorithm>

namespace msd {
namespace bwdk {

typedef float mfma4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kChanBlock = 16;

template <int V> struct XTile {
    static constexpr int kVox = kWave * V;        // voxels per wave
    static constexpr int kStride = kVox + 4;      // floats per channel row (bank spread for the b128 reads)
    static constexpr int kFloats = kChanBlock * kStride;
};

template <int NDIM, bool RELU, int V, int NCB>
__global__ __launch_bounds__(kThreads, 2) void bwdk_mfma(Geom g, RowTeams rt, int remap, int tiles_per_wg, int ntiles,
                                                      int groups_per_image, View<const float> out,
                                                      View<const float> gy, View<const float> x,
                                                      float *__restrict__ part, int want_bias)
{
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K, NPQ = RowTaps<NDIM>::NPQ;
    constexpr int TG = NDIM == 3 ? 2 : 1;         // groups of 16 tap rows
    constexpr int NS = 4 * V;                     // 16-voxel MFMA groups per wave
    const int tid = threadIdx.x;
    const int wave = tid / kWave, wl = tid % kWave;
    const int team = tid / rt.lpr, lane = tid % rt.lpr;
    const int mk = wl / 16, mj = wl % 16;         // MFMA k (voxel) and i/j (tap or channel) of this lane

    // LDS: while a tile is set up, S (staged rows) and AL (taps x voxels); in
    // the channel loop the same memory holds the wave-private input tiles XS.
    constexpr int TVP = kThreads * V + 4;         // AL row stride (bank spread for the b128 reads)
    float *S = lds;
    float *AL = lds + (size_t)NPQ * kThreads * V;
    float *XS = lds + (size_t)wave * XTile<V>::kFloats;

    const int co = blockIdx.z % g.Wd;
    const int chunk = blockIdx.z / g.Wd;
    const int c0 = chunk * NCB * kChanBlock;
    const int ones_ch = want_bias ? g.C : -1;     // virtual channel of ones -> bias sum
    const int c_end = min(g.C + (want_bias ? 1 : 0), c0 + NCB * kChanBlock);

    mfma4 D[NCB][TG];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++) D[cb][tg] = mfma4{0.f, 0.f, 0.f, 0.f};

    const int lb = block_for_xcd(blockIdx.x, gridDim.x, remap);
    View<const float> out_c = out, gy_c = gy;
    out_c.p = RELU ? out.p + (int64_t)co * out.sc : nullptr;
    gy_c.p = gy.p + (int64_t)co * gy.sc;

    for (int ti = 0; ti < tiles_per_wg; ti++) {
        const int tile = lb * tiles_per_wg + ti;
        if (tile >= ntiles) break;                // uniform over the workgroup
        int64_t xsc = x.sc;
        asm volatile("" : "+s"(xsc));             // keeps the 16 channel offsets from being hoisted out of the loop
        const int b = tile / groups_per_image;
        const int row0 = (tile % groups_per_image) * rt.rpw;
        const int row = row0 + team;
        const int x0 = lane * V;
        const bool act = row < rt.nrows && x0 < g.W;
        const int rr = min(row, rt.nrows - 1);

        const float *xp0 = x.p + (int64_t)b * x.sb + (int64_t)(rr / g.H) * x.sz + (int64_t)(rr % g.H) * x.sy +
                           min(x0, g.W - V);
        const int ncb = (c_end - c0 + kChanBlock - 1) / kChanBlock;
        // Input values of 16 channels for this lane's voxels.  Branch-free: every
        // lane loads from a clamped, valid address, so all 16 loads are in flight
        // together; values that must not count are replaced in fix_block().
        float xv[kChanBlock][V];
        auto load_block = [&](int cb) {
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
        load_block(0);   // issued ahead of the set-up so its latency overlaps with it

        {
            float own[1][NPQ][V];
            float *srows = S + (size_t)team * NPQ * V * rt.lpr;
            stage_source_rows<NDIM, RELU, 1, V>(g, rt, out_c, gy_c, b, rr / g.H, rr % g.H, lane, act, srows, own);
            // the K taps of this lane's V voxels -> AL[tap][tid * V + i]
            float t[NPQ][3][V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                const SideTaps<V> side(x0 + i, g.W, g.dil, rt.lpr);
#pragma unroll
                for (int pq = 0; pq < NPQ; pq++) {
                    side.read(srows + (size_t)pq * V * rt.lpr, t[pq][0][i], t[pq][2][i]);
                    t[pq][1][i] = own[0][pq][i];
                }
            }
#pragma unroll
            for (int pq = 0; pq < NPQ; pq++)
#pragma unroll
                for (int r = 0; r < 3; r++) {
#pragma unroll
                    for (int i = 0; i < V; i++) t[pq][r][i] = act ? t[pq][r][i] : 0.f;
                    store_vec<V>(AL + (size_t)(pq * 3 + r) * TVP + tid * V, t[pq][r]);
                }
        }
        __syncthreads();
        // A operands: a[tg][s][e] = A[tap = tg*16 + mj](voxel wave*64V + 16 s + 4 mk + e)
        float a[TG][NS][4];
#pragma unroll
        for (int tg = 0; tg < TG; tg++) {
            const int tap = tg * 16 + mj;
            const float *arow = AL + (size_t)min(tap, K - 1) * TVP + wave * XTile<V>::kVox + 4 * mk;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const f32x4 av = *reinterpret_cast<const f32x4 *>(arow + 16 * s);
#pragma unroll
                for (int e = 0; e < 4; e++) a[tg][s][e] = tap < K ? av[e] : 0.f;
            }
        }
        __syncthreads();   // S and AL are dead from here on: the channel loop reuses their memory

        // runtime loop: unrolled, the per-channel addresses and predicates of all
        // NCB blocks would be computed up front and spill
#pragma unroll 1
        for (int cb = 0; cb < ncb; cb++) {
            // this wave's 64*V voxels of 16 channels -> wave-private LDS tile [channel][voxel]
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
        __syncthreads();   // all waves are done with their tiles before the next set-up reuses the memory
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
        if (col < nk)
            gk[col] += s;
        else
            gb[col - nk] += s;
    }
}

constexpr size_t kMaxLds = 160 * 1024;   // LDS per CU on gfx950; above 64 KB a kernel must opt in

template <int NDIM, int V, int NCB>
size_t lds_bytes()
{
    constexpr int TG = NDIM == 3 ? 2 : 1;
    const size_t setup = ((size_t)RowTaps<NDIM>::NPQ * kThreads * V + (size_t)Taps<NDIM>::K * (kThreads * V + 4)) * 4;
    const size_t main_loop = (size_t)kWaves * XTile<V>::kFloats * 4;
    const size_t epilogue = (size_t)kWaves * NCB * TG * 4 * kWave * 4;
    return std::max(setup, std::max(main_loop, epilogue));
}

template <int NDIM, bool RELU, int V, int NCB>
hipError_t launch(const Geom &g, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    constexpr int K = Taps<NDIM>::K;
    RowTeams rt;
    make_row_teams(g, V, &rt);
    const int groups = (rt.nrows + rt.rpw - 1) / rt.rpw;
    const int ntiles = groups * g.B;
    const int remap = knob(kKnobXcdRemap, 1);
    int wgs = min(ntiles, knob(kKnobBwdkBlocks, kMaxPartialRows));
    wgs = min(wgs, kMaxPartialRows);
    const int tiles_per_wg = (ntiles + wgs - 1) / wgs;
    wgs = (ntiles + tiles_per_wg - 1) / tiles_per_wg;
    const int rows = remap ? xcd_grid(wgs) : wgs;   // padding workgroups write zero rows
    if (rows > kMaxPartialRows) return hipErrorInvalidConfiguration;
    const int want_bias = gb != nullptr;
    const int chunks = (g.C + want_bias + NCB * kChanBlock - 1) / (NCB * kChanBlock);
    const size_t lds = lds_bytes<NDIM, V, NCB>();
    if (lds > 64 * 1024) {
        static const hipError_t attr = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&bwdk_mfma<NDIM, RELU, V, NCB>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
        if (attr != hipSuccess) return attr;
    }
    hipLaunchKernelGGL((bwdk_mfma<NDIM, RELU, V, NCB>), dim3(rows, 1, chunks * g.Wd), dim3(kThreads), lds, s, g, rt,
                       remap, tiles_per_wg, ntiles, groups, out, gy, x, ws, want_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nk = (int64_t)g.Wd * g.C * K;
    const int64_t ncols = nk + (want_bias ? g.Wd : 0);
    hipLaunchKernelGGL(reduce_columns, dim3((ncols + 3) / 4), dim3(256), 0, s, ws, rows, nk, ncols, gk, gb);
    return hipGetLastError();
}

template <int NDIM, bool RELU, int V>
hipError_t pick_ncb(const Geom &g, const View<const float> &out, const View<const float> &gy,
                    const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    const int need = (g.C + (gb != nullptr) + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch<NDIM, RELU, V, 1>(g, out, gy, x, gk, gb, ws, s);
    if (need <= 2) return launch<NDIM, RELU, V, 2>(g, out, gy, x, gk, gb, ws, s);
    if (need <= 4) return launch<NDIM, RELU, V, 4>(g, out, gy, x, gk, gb, ws, s);
    return launch<NDIM, RELU, V, 8>(g, out, gy, x, gk, gb, ws, s);
}

// Voxels per lane: V-wide accesses aligned in every view and a tile of
// 256 * V voxels made of whole rows (row-team mapping with 256 lanes).
template <int NDIM>
int choose_vec(const Geom &g, bool relu, int vmax, const View<const float> &out, const View<const float> &gy,
               const View<const float> &x)
{
    for (int v = 4; v >= 1; v /= 2) {
        if (v > vmax) continue;
        if (!rows_aligned(x, g.W, v) || !rows_aligned(gy, g.W, v) || (relu && !rows_aligned(out, g.W, v))) continue;
        RowTeams rt;
        if (!make_row_teams(g, v, &rt) || rt.lpr * rt.rpw != kThreads) continue;
        return v;
    }
    return 0;
}

template <int NDIM>
bool supported_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x)
{
    if (x.sx != 1 || gy.sx != 1 || (relu && out.sx != 1)) return false;
    return choose_vec<NDIM>(g, relu, 4, out, gy, x) != 0;
}

template <int NDIM, bool RELU>
hipError_t pick_vec(const Geom &g, const View<const float> &out, const View<const float> &gy,
                    const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    const int vmax = knob(NDIM == 3 ? kKnobBwdkVec3d : kKnobBwdkVec2d, NDIM == 3 ? 2 : 4);
    int v = choose_vec<NDIM>(g, RELU, vmax, out, gy, x);
    if (v == 0) v = choose_vec<NDIM>(g, RELU, 4, out, gy, x);
    if (v == 4) return pick_ncb<NDIM, RELU, 4>(g, out, gy, x, gk, gb, ws, s);
    if (v == 2) return pick_ncb<NDIM, RELU, 2>(g, out, gy, x, gk, gb, ws, s);
    if (v == 1) return pick_ncb<NDIM, RELU, 1>(g, out, gy, x, gk, gb, ws, s);
    return hipErrorInvalidConfiguration;
}

template <int NDIM>
hipError_t run_nd(const Geom &g, bool relu, const View<const float> &out, const View<const float> &gy,
                  const View<const float> &x, float *gk, float *gb, float *ws, hipStream_t s)
{
    return relu ? pick_vec<NDIM, true>(g, out, gy, x, gk, gb, ws, s)
                : pick_vec<NDIM, false>(g, out, gy, x, gk, gb, ws, s);
}

}  // namespace bwdk
}  // namespace msd
