// Forward pass for fp32 with unit x-stride and one or two output channels:
//     out[v] = [max(0, .)] ( bias + sum_ci sum_{p,q,r} x[ci][fold(v + dil*(p,q,r))] * k[ci][p][q][r] )
//
// Work split.  A team of `lpr` lanes (a multiple of 64) owns full image rows,
// V consecutive voxels per lane.  One workgroup computes a small lattice of
// RZ x RY output rows whose members are dil apart in z and y:
//     rows (z0 + jz*dil, y0 + jy*dil),  jz < RZ, jy < RY.
// Their 3x3 (x3) taps fall on the (RZ+2) x (RY+2) input rows of the same
// lattice, so each input row that is loaded serves up to nine output rows from
// registers (an ordinary square tile would need a halo of 2*dil rows).
// Along x nothing is shifted in the channel loop at all: for every output row
// the lane accumulates the three partial sums
//     T_r[x'] = sum_ci sum_{p,q} x[ci][..][x'] * k[ci][p][q][r],      r = 0, 1, 2
// at its own positions x', and the row is finished once, after the channel
// loop, as  out[x] = T_0[fold(x - dil)] + T_1[x] + T_2[fold(x + dil)]  through LDS.
// The channel loop is therefore: one aligned V-wide load per input row, then
// 3*V fused multiply-adds per (output row, tap row) pair, with wave-uniform
// weights from scalar registers.
//
// The input channels are split over KS groups of lanes of the workgroup
// (channel ci goes to group ci % KS), which multiplies the number of waves in
// flight; the groups' partial sums meet in LDS in the finishing step, in a fixed order.
// Algorithmic traffic: (C + w) * N * 4 bytes.
#pragma once
#include "msd_kernels.h"
#include "msd_rows.h"

namespace msd {
namespace fwd {

constexpr int kOrder = 4;   // edge of the (y, z) blocks the 3D tiles are numbered in

struct Lattice {
    int lpr;        // lanes per row
    int ks;         // channel groups per workgroup
    int segs_y;     // lattice segments per y residue
    int segs_z;
    int tiles_y;    // dil * segs_y
    int tiles_z;    // dil * segs_z (1 in 2D)
    int ntiles;
    int by_class;   // 3D: tiles numbered residue class by residue class (2: a class row by row, no blocks)
};

// First output row (y0, z0) of the lattice this workgroup computes; false for the padding
// blocks of the grid and for lattices that start past the image (uniform over the workgroup).
template <int NDIM, int RZ, int RY>
__device__ __forceinline__ bool tile_origin(const Geom &g, const Lattice &lt, int remap, int &y0, int &z0)
{
    const int tile = block_for_xcd(blockIdx.x, gridDim.x, remap);
    if (tile >= lt.ntiles) return false;         // padding block
    // 3D: tiles are numbered in blocks of kOrder x kOrder (y, z) neighbours.  Neighbouring
    // lattices share a third of their input rows, and only tiles that start together walk the
    // channels in step and find each other's rows in the L2.
    int ty, tz;
    if (NDIM == 3 && lt.by_class == 2) {
        // small classes (large dilations): all lattices of a class are resident together
        // anyway, so they are simply numbered row by row, with no padding of the grid
        const int per_class = lt.segs_y * lt.segs_z;
        const int cls = tile / per_class, rem = tile % per_class;
        ty = (cls % g.dil) * lt.segs_y + rem % lt.segs_y;
        tz = (cls / g.dil) * lt.segs_z + rem / lt.segs_y;
    } else if (NDIM == 3 && lt.by_class) {
        // An input row feeds only output rows of its own residue class (y mod dil, z mod dil):
        // the lattices of one class share all their input, those of different classes nothing.
        // So the classes are numbered one after the other, and inside a class the lattices in
        // blocks of kOrder x kOrder neighbours: what runs together, on one XCD, reads the same
        // rows, and the L2 serves the re-reads.
        const int bys = (lt.segs_y + kOrder - 1) / kOrder, bzs = (lt.segs_z + kOrder - 1) / kOrder;
        const int per_class = bys * bzs * kOrder * kOrder;
        const int cls = tile / per_class, rem = tile % per_class;
        const int blk = rem / (kOrder * kOrder), within = rem % (kOrder * kOrder);
        const int sy = (blk % bys) * kOrder + within % kOrder, sz = (blk / bys) * kOrder + within / kOrder;
        if (sy >= lt.segs_y || sz >= lt.segs_z) return false;   // padding of the block grid
        ty = (cls % g.dil) * lt.segs_y + sy;
        tz = (cls / g.dil) * lt.segs_z + sz;
    } else if (NDIM == 3) {
        const int blk = tile / (kOrder * kOrder), within = tile % (kOrder * kOrder);
        const int nby = (lt.tiles_y + kOrder - 1) / kOrder;
        ty = (blk % nby) * kOrder + within % kOrder;
        tz = (blk / nby) * kOrder + within / kOrder;
        if (ty >= lt.tiles_y || tz >= lt.tiles_z) return false;   // padding of the block grid
    } else {
        ty = tile;
        tz = 0;
    }
    y0 = ty / lt.segs_y + (ty % lt.segs_y) * RY * g.dil;
    z0 = NDIM == 3 ? tz / lt.segs_z + (tz % lt.segs_z) * RZ * g.dil : 0;
    return y0 < g.H && z0 < g.D;                 // false: empty tail of a residue class
}

template <int NDIM, bool RELU, int WOUT, int V, int RZ, int RY>
__global__ __launch_bounds__(NDIM == 3 ? 512 : 1024, (NDIM == 3 && V == 1 && WOUT == 1) ? (RZ * RY > 9 ? 4 : 8) : 1) void fwd_lattice(Geom g, Lattice lt, int remap, View<const float> x,
                                                    const float *__restrict__ k, const float *__restrict__ bias,
                                                    View<float> out)
{
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K;
    constexpr int NZ = Taps<NDIM>::NZ;          // z taps: 3 or 1
    constexpr int LZ = NDIM == 3 ? RZ + 2 : 1;  // input lattice levels along z
    constexpr int LY = RY + 2;
    static_assert(NDIM == 3 || RZ == 1, "2D has a single z level");

    int y0, z0;
    if (!tile_origin<NDIM, RZ, RY>(g, lt, remap, y0, z0)) return;   // padding block or empty tail (whole workgroup)

    const int lane = threadIdx.x % lt.lpr;
    const int kg = __builtin_amdgcn_readfirstlane(threadIdx.x / lt.lpr);   // uniform: lpr is a multiple of 64
    const int x0 = min(lane * V, g.W - V);       // lanes past the row load a valid address; nothing is stored
    const bool act = lane * V < g.W;
    const int b = blockIdx.y;

    // valid output rows of this lattice (the rest lie past the image edge)
    const int nyv = min(RY, (g.H - y0 + g.dil - 1) / g.dil);
    const int nzv = NDIM == 3 ? min(RZ, (g.D - z0 + g.dil - 1) / g.dil) : 1;

    // Offsets of the input lattice rows (folded at the image edges).  Lattice levels past
    // nyv + 1 (nzv + 1) feed only output rows outside the image: they repeat the last level
    // that is needed, so that their loads hit the cache instead of fetching rows nobody uses.
    // A load address is a wave-uniform base (batch, channel, z level: scalar registers and
    // scalar arithmetic) plus a 32-bit byte offset per lane (y row and x position, computed
    // once), so the channel loop spends no vector instructions on it.
    int64_t offz[LZ];
    uint32_t offyx[LY];
#pragma unroll
    for (int m = 0; m < LZ; m++)
        offz[m] = NDIM == 3 ? (int64_t)min(reflect_idx(min(z0 + (min(m, nzv + 1) - 1) * g.dil, 2 * g.D - 1), g.D), g.D - 1) * x.sz * 4 : 0;
#pragma unroll
    for (int m = 0; m < LY; m++)
        offyx[m] = 4u * (uint32_t)(min(reflect_idx(min(y0 + (min(m, nyv + 1) - 1) * g.dil, 2 * g.H - 1), g.H), g.H - 1) * (int)x.sy + x0);

    float acc[WOUT][RZ][RY][3][V];
#pragma unroll
    for (int co = 0; co < WOUT; co++)
#pragma unroll
        for (int jz = 0; jz < RZ; jz++)
#pragma unroll
            for (int jy = 0; jy < RY; jy++)
#pragma unroll
                for (int r = 0; r < 3; r++)
#pragma unroll
                    for (int i = 0; i < V; i++) acc[co][jz][jy][r][i] = 0.f;

    const char *xb = reinterpret_cast<const char *>(x.p + (int64_t)b * x.sb);
    for (int cn = kg; cn < g.C; cn += lt.ks) {
        const int ci = g.reverse ? g.C - 1 - cn : cn;
        const char *xc = xb + (int64_t)ci * x.sc * 4;
        float w[WOUT][K];
#pragma unroll
        for (int co = 0; co < WOUT; co++)
#pragma unroll
            for (int t = 0; t < K; t++) w[co][t] = k[((int64_t)co * g.C + ci) * K + t];
        // (redefining the lane offsets here keeps their widening to 64 bits inside the loop, next
        // to the loads, where it costs nothing; hoisted, it would turn them into register pairs
        // and every load address into a 64-bit vector addition)
#pragma unroll
        for (int my = 0; my < LY; my++) asm volatile("" : "+v"(offyx[my]));
        // all row loads of this channel are issued before the first multiply-add
        float xv[LZ][LY][V];
#pragma unroll
        for (int mz = 0; mz < LZ; mz++) {
            uint64_t xz = reinterpret_cast<uint64_t>(xc + offz[mz]);
            asm volatile("" : "+s"(xz));          // stays a scalar base: the loads take it beside the lane offset
#pragma unroll
            for (int my = 0; my < LY; my++) load_global_vec<V>(xz, offyx[my], xv[mz][my]);
        }
        if constexpr (WOUT == 1) __builtin_amdgcn_sched_barrier(0);
        // output rows past the image edge (partial lattices) are skipped, uniformly per workgroup
#pragma unroll
        for (int jz = 0; jz < RZ; jz++) {
            if (jz >= nzv) break;
#pragma unroll
            for (int jy = 0; jy < RY; jy++) {
                if (jy >= nyv) break;
#pragma unroll
                for (int p = 0; p < NZ; p++)
#pragma unroll
                    for (int q = 0; q < 3; q++)
#pragma unroll
                        for (int co = 0; co < WOUT; co++)
#pragma unroll
                            for (int r = 0; r < 3; r++) {
                                const float wv = w[co][(p * 3 + q) * 3 + r];
#pragma unroll
                                for (int i = 0; i < V; i++)
                                    acc[co][jz][jy][r][i] += xv[NDIM == 3 ? jz + p : 0][jy + q][i] * wv;
                            }
            }
        }
    }

    // Finish the rows one at a time.  LDS holds T_r of the current row for every
    // channel group: T[kg][r][staged x]; group (row counter % KS) adds the groups
    // up at the three shifted positions and writes the row.
    const int rowlen = V * lt.lpr;
    float *T = lds;
    int counter = 0;
#pragma unroll
    for (int co = 0; co < WOUT; co++) {
        const float bv = bias[co];
#pragma unroll
        for (int jz = 0; jz < RZ; jz++)
#pragma unroll
            for (int jy = 0; jy < RY; jy++) {
                const int z = z0 + jz * g.dil, y = y0 + jy * g.dil;
                if (z >= g.D || y >= g.H) continue;             // uniform over the workgroup
#pragma unroll
                for (int r = 0; r < 3; r++)
#pragma unroll
                    for (int i = 0; i < V; i++)
                        T[(kg * 3 + r) * rowlen + i * lt.lpr + lane] = act ? acc[co][jz][jy][r][i] : 0.f;
                __syncthreads();
                if (kg == counter % lt.ks && act) {
                    float o[V];
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        const int xx = x0 + i;
                        const int i0 = staged_index<V>(reflect_idx(xx - g.dil, g.W), lt.lpr);
                        const int i1 = i * lt.lpr + lane;
                        const int i2 = staged_index<V>(reflect_idx(xx + g.dil, g.W), lt.lpr);
                        float s = bv;
                        for (int kk = 0; kk < lt.ks; kk++) {
                            const float *tk = T + (size_t)kk * 3 * rowlen;
                            s += tk[i0] + tk[rowlen + i1] + tk[2 * rowlen + i2];
                        }
                        o[i] = RELU ? (s > 0.f ? s : 0.f) : s;
                    }
                    store_vec<V>(out.p + (int64_t)b * out.sb + (int64_t)co * out.sc + (int64_t)z * out.sz +
                                     (int64_t)y * out.sy + x0,
                                 o);
                }
                counter++;
                __syncthreads();
            }
    }
}

constexpr size_t kMaxLds = 64 * 1024;

// 2D: while the input channels of a layer fit the 256 MB memory-side cache, one voxel per lane
// (a row of 1024 lanes, 16 waves per CU) is 8-15 % faster than four (8 waves): the loads come
// back sooner than from memory and more waves keep more of them in flight.  Past that size
// the wider loads win by as much (1024 x 1024, 60 against 70 channels).
constexpr int64_t kCacheResidentBytes = 256 * 1000 * 1000;

// Threads of a workgroup (the kernel's launch bound): a row of W / V lanes must fit.
inline int max_lanes(int ndim) { return ndim == 3 ? 512 : 1024; }

inline bool make_lattice(const Geom &g, int V, int rz, int ry, int ks_wanted, Lattice *lt)
{
    const int need = (g.W + V - 1) / V;
    const int lpr = (need + kWave - 1) / kWave * kWave;
    // 3D: at most 8 waves per workgroup, so that several workgroups share a CU and their
    // phases (loads, arithmetic, LDS epilogue) overlap; long rows then split less
    const int max_threads = max_lanes(g.ndim);
    if (lpr > max_threads) return false;
    int ks = ks_wanted;
    while (ks > 1 && (ks * lpr > max_threads || ks > g.C)) ks /= 2;
    if ((size_t)ks * 3 * V * lpr * sizeof(float) > kMaxLds) return false;
    lt->lpr = lpr;
    lt->ks = ks;
    lt->segs_y = ((g.H + g.dil - 1) / g.dil + ry - 1) / ry;
    lt->tiles_y = g.dil * lt->segs_y;
    if (g.ndim == 3) {
        lt->segs_z = ((g.D + g.dil - 1) / g.dil + rz - 1) / rz;
        lt->tiles_z = g.dil * lt->segs_z;
        lt->by_class = knob(kKnobFwdClass3d, 1);
        if (lt->by_class && lt->segs_y * lt->segs_z <= 128) lt->by_class = 2;
        if (lt->by_class == 2)
            lt->ntiles = g.dil * g.dil * lt->segs_y * lt->segs_z;
        else if (lt->by_class)
            lt->ntiles = g.dil * g.dil * ((lt->segs_y + kOrder - 1) / kOrder) * ((lt->segs_z + kOrder - 1) / kOrder) *
                         kOrder * kOrder;
        else
            lt->ntiles = ((lt->tiles_y + kOrder - 1) / kOrder) * ((lt->tiles_z + kOrder - 1) / kOrder) * kOrder * kOrder;
    } else {
        lt->by_class = 0;
        lt->segs_z = 1;
        lt->tiles_z = 1;
        lt->ntiles = lt->tiles_y;
    }
    return true;
}

template <int NDIM, bool RELU, int WOUT, int V, int RZ, int RY>
hipError_t launch(const Geom &g, const View<const float> &x, const float *k, const float *bias,
                  const View<float> &out, hipStream_t s)
{
    Lattice lt;
    if (!make_lattice(g, V, RZ, RY, knob(kKnobFwdSplit, 2), &lt)) return hipErrorInvalidConfiguration;
    const int remap = knob(kKnobXcdRemap, 1);
    const dim3 grid(remap ? xcd_grid(lt.ntiles) : lt.ntiles, g.B, 1);
    const size_t lds = (size_t)lt.ks * 3 * V * lt.lpr * sizeof(float);
    hipLaunchKernelGGL((fwd_lattice<NDIM, RELU, WOUT, V, RZ, RY>), grid, dim3(lt.ks * lt.lpr), lds, s, g, lt, remap, x,
                       k, bias, out);
    return hipGetLastError();
}

// Largest V whose accesses are aligned in both views and that leaves at least
// one full wave per row.
inline int choose_vec(const Geom &g, int vmax, const View<const float> &x, const View<float> &out)
{
    for (int v = 4; v >= 1; v /= 2) {
        if (v > vmax) continue;
        if (!rows_aligned(x, g.W, v) || !rows_aligned(out, g.W, v)) continue;
        if (v > 1 && (g.W + v - 1) / v < kWave) continue;   // keep the lanes of a wave busy
        if ((g.W + v - 1) / v > max_lanes(g.ndim)) continue;
        return v;
    }
    return 0;
}

template <int NDIM>
bool supported_nd(const Geom &g, const View<const float> &x, const View<float> &out)
{
    if (g.Wd > 2 || x.sx != 1 || out.sx != 1) return false;
    if ((int64_t)(g.H - 1) * x.sy + g.W >= ((int64_t)1 << 30)) return false;   // 32-bit in-plane byte offsets
    if (g.W < 32) return false;                  // rows shorter than half a wave: the generic kernel does better
    return choose_vec(g, 4, x, out) != 0;
}

// 2D, one output channel: the instance with `ry` output rows per tile (2 to 6; 4 otherwise).
template <bool RELU, int V>
hipError_t launch_rows_2d(int ry, const Geom &g, const View<const float> &x, const float *k, const float *bias,
                          const View<float> &out, hipStream_t s)
{
    switch (ry) {
    case 2: return launch<2, RELU, 1, V, 1, 2>(g, x, k, bias, out, s);
    case 3: return launch<2, RELU, 1, V, 1, 3>(g, x, k, bias, out, s);
    case 5: return launch<2, RELU, 1, V, 1, 5>(g, x, k, bias, out, s);
    case 6: return launch<2, RELU, 1, V, 1, 6>(g, x, k, bias, out, s);
    default: return launch<2, RELU, 1, V, 1, 4>(g, x, k, bias, out, s);
    }
}

template <int NDIM, bool RELU, int WOUT>
hipError_t pick(const Geom &g, const View<const float> &x, const float *k, const float *bias, const View<float> &out,
                hipStream_t s)
{
    int vmax = knob(NDIM == 3 ? kKnobFwdVec3d : kKnobFwdVec2d, NDIM == 3 ? 1 : 4);
    const bool resident = (int64_t)g.B * g.C * x.sc * (int64_t)sizeof(float) <= kCacheResidentBytes;
    if (NDIM == 2 && WOUT == 1 && knob(kKnobFwdVec2d, -1) < 0 && resident) vmax = 1;
    int v = choose_vec(g, vmax, x, out);
    if (v == 0) v = choose_vec(g, 4, x, out);
    if constexpr (NDIM == 3) {
        if (v == 4) return launch<3, RELU, WOUT, 4, 2, 2>(g, x, k, bias, out, s);
        if (v == 2) return launch<3, RELU, WOUT, 2, 2, 4>(g, x, k, bias, out, s);
        if (v == 1) {
            if constexpr (WOUT == 1) {
                // Lattices of 3 x 3 rows instead of 2 x 4 where they cover the residue classes
                // with at least 1/16 fewer tiles (a partly filled lattice costs as much time as a
                // full one): at 128^3 dilations 3, 5, 9, 10, by 2 to 12 %.  Not at dilations 1
                // and 2, where the nine rows per tile cost more than the fewer tiles save.
                const int rows_y = (g.H + g.dil - 1) / g.dil, rows_z = (g.D + g.dil - 1) / g.dil;
                const long t24 = (long)((rows_z + 1) / 2) * ((rows_y + 3) / 4);
                const long t33 = (long)((rows_z + 2) / 3) * ((rows_y + 2) / 3);
                // Lattices of 4 x 4 rows read 36 input rows for 16 output rows (2.25 per row
                // instead of 3) and halve the number of tiles; they take twice the registers, so
                // two workgroups fewer share a CU.
                const long t44 = (long)((rows_z + 3) / 4) * ((rows_y + 3) / 4);
                const int forced = knob(kKnobFwdLattice3d, 0);
                if (forced == 44) return launch<3, RELU, 1, 1, 4, 4>(g, x, k, bias, out, s);
                if (forced == 33) return launch<3, RELU, 1, 1, 3, 3>(g, x, k, bias, out, s);
                if (forced == 24) return launch<3, RELU, 1, 1, 2, 4>(g, x, k, bias, out, s);
                (void)t44;
                if (g.dil >= 3 && t33 * 16 < t24 * 15) return launch<3, RELU, 1, 1, 3, 3>(g, x, k, bias, out, s);
            }
            return launch<3, RELU, WOUT, 1, 2, 4>(g, x, k, bias, out, s);
        }
    } else {
        if constexpr (WOUT == 1) {
            // Rows per tile: all tiles cost the same, so the time is (rounds of tiles over
            // the 256 CUs) x (rows per tile); with few tiles a longer chain that avoids a
            // nearly empty last round wins.  Tiles of 2 or 3 rows read 2 and 1.67 input rows
            // per output row instead of 1.5 and less: they are candidates only for images so
            // small that tiles of four rows leave CUs idle, and while the input comes from
            // the cache (256 x 256, 100 channels: 16 against 21 us).
            const long tiles4 = (long)g.dil * (((g.H + g.dil - 1) / g.dil + 3) / 4) * g.B;
            const int first = resident && tiles4 < 256 ? 2 : 4;
            int best = first;
            long best_cost = 0;
            for (int ry = first; ry <= 6; ry++) {
                const long tiles = (long)g.dil * (((g.H + g.dil - 1) / g.dil + ry - 1) / ry) * g.B;
                const long cost = (tiles + 255) / 256 * ry;
                if (ry == first || cost < best_cost) { best = ry; best_cost = cost; }
            }
            best = knob(kKnobFwdRows2d, best);
            if (v == 4) return launch_rows_2d<RELU, 4>(best, g, x, k, bias, out, s);
            if (v == 2) return launch_rows_2d<RELU, 2>(best, g, x, k, bias, out, s);
            if (v == 1) return launch_rows_2d<RELU, 1>(best, g, x, k, bias, out, s);
        } else {
            // two output channels double the accumulators: three rows per tile keep them in registers
            if (v == 4) return launch<2, RELU, 2, 4, 1, 3>(g, x, k, bias, out, s);
            if (v == 2) return launch<2, RELU, 2, 2, 1, 4>(g, x, k, bias, out, s);
            if (v == 1) return launch<2, RELU, 2, 1, 1, 4>(g, x, k, bias, out, s);
        }
    }
    return hipErrorInvalidConfiguration;
}

template <int NDIM>
hipError_t run_nd(const Geom &g, bool relu, const View<const float> &x, const float *k, const float *bias,
                  const View<float> &out, hipStream_t s)
{
    if (g.Wd == 1)
        return relu ? pick<NDIM, true, 1>(g, x, k, bias, out, s) : pick<NDIM, false, 1>(g, x, k, bias, out, s);
    return relu ? pick<NDIM, true, 2>(g, x, k, bias, out, s) : pick<NDIM, false, 2>(g, x, k, bias, out, s);
}

}  // namespace fwd
}  // namespace msd
