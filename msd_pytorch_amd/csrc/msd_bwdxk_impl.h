// backward_x and backward_k (+ bias) of one layer in a single pass over the input
// channels, fp32, unit x-stride, output gradient already masked:
//     grad_input[ci][u] += sum_t k[ci][t] * A[t](u)
//     grad_kernel[ci][t] += sum_u x[ci][u] * A[t](u),     grad_bias += sum_u A[centre](u)
// for one output channel, or summed over / repeated for two or three (2D): the output
// channels of one layer, or two or three one-channel layers of a dense block with their own
// dilations, weights and gradients, which share the input channels of the lowest of them.
// Both need the same adjoint-form gather A[t](u) of the output gradient (msd_adjoint.h,
// msd_rows.h); done once per tile of rows, it then serves a stream over the input
// channels that reads x[ci], reads and writes grad_input[ci], and touches nothing else.
//
// Work split.  Row teams as in msd_rows.h: a team of lpr lanes (a multiple of 64 here)
// owns an image row, a lane V consecutive voxels of it, so a WAVE owns 64*V consecutive
// voxels.  After the gather every lane holds A[t] of its own voxels in registers
// ("voxel layout"): that is what the grad_input update needs, K*V fused multiply-adds
// per channel with wave-uniform weights.  The weight gradient is a contraction over
// voxels and goes to the matrix cores, v_mfma_f32_16x16x4_f32 with taps as rows,
// 16 input channels as columns and 4 voxels per instruction:
//   A operand  the wave writes its A[t][voxel] tile to a private LDS tile once per row
//              tile and reads 4-voxel groups of row `tap` back per instruction;
//   B operand  lane (channel j, voxel group k) loads x[c0 + j][16 s + 4 k ...+3] straight
//              from memory as one 16-byte access: the layout change costs nothing.
// The channel loop is software-pipelined in stages of 16 to 64 of the wave's voxels for
// 16 channels of x plus 2 to 8 channels of grad_input: the loads of the next stage are
// issued before the arithmetic of the current one, into the other of two register sets.
// Partial sums of the weight gradient stay in registers over all row tiles of a
// workgroup, are added over its waves in LDS and leave as one column-major row per
// workgroup; bwdk::reduce_columns adds the rows in a fixed order.
//
// Registers.  Kernel arguments live in scalar registers for the whole kernel, so they
// are kept small: 32-bit strides (checked on the host), no view that is not read.
// grad_input is addressed as a wave-uniform channel base plus a 32-bit lane offset, which
// costs no vector registers or vector arithmetic per channel.
// Algorithmic traffic: (3C + 2w) * N * 4 bytes.
#pragma once
#include "msd_bwdk_impl.h"

#include <atomic>
#include <type_traits>

#ifndef MSD_XPAIR
#define MSD_XPAIR 1
#endif
#ifndef MSD_INNER_PATH
#define MSD_INNER_PATH 1
#endif
#ifndef MSD_PIPELINE_SETS_EXPR
#define MSD_PIPELINE_SETS_EXPR 2
#endif

namespace msd {
namespace bwdxk {

using bwdk::kChanBlock;
using bwdk::kThreads;
using bwdk::kWaves;
using bwdk::mfma4;

// Wave-private LDS tile [output channel][tap][voxel]; one more row of zeros feeds the MFMA
// rows past the last tap.
template <int NDIM, int V, int WOUT> struct ATile {
    static constexpr int kStride = kWave * V + 4;     // floats per row (bank spread for the b128 reads)
    static constexpr int kRows = WOUT * Taps<NDIM>::K + 1;
    static constexpr int kFloats = kRows * kStride;
};

// Element strides {batch, channel, z, y} of a tensor; the x stride is 1.
struct Plane {
    int sb, sc, sz, sy;
};

// One step of a workgroup from tile to tile (group_step tiles ahead), taken apart on the host so
// that the kernel advances its position with additions and compares only: in segments of a row,
// row groups of an image and batch items; the row groups again as rows, split into y and z; and
// the rows of a wrap to the next batch item (ngroups * rpw) and of a carried segment (rpw).
struct TileStep {
    int seg, gi, b;
    int y, z;
    int wrap_y, wrap_z;
    int carry_y, carry_z;
};

struct Args {
    Geom g;
    RowTeams rt;
    int remap, tiles_per_wg, ngroups, total_groups;
    int group_step;      // 1: a workgroup walks consecutive row groups; > 1: every group_step-th one
    Plane gy;            // masked output gradient, one to three channels
    Plane x;             // input channels
    Plane gx;            // grad_input channels (written through a cast)
    int mask_from;       // activations (viewed like grad_input) mask the channels >= mask_from
    int want_bias;
    RowSegments sg;      // LONG instances
    UpperDilations up;   // layers of a dense block in one pass: the dilations of output channels 1 and 2
    TileStep step;
};

// The waves' tiles share the LDS of the staged rows (two outputs at four voxels per lane: the
// tiles alone are 79 KB; three outputs, or 3D at two voxels per lane: 59 KB).
template <int NDIM, int V, int WOUT>
constexpr bool tiles_over_staging() { return (NDIM == 2 && ((V == 4 && WOUT == 2) || WOUT == 3)) || (NDIM == 3 && (V == 2 || WOUT >= 2)); }

// Workgroups (of four waves) that are resident per CU.  The 3D kernel with one voxel per lane
// (pipeline stages of 16 voxels, arguments read again per tile, row arithmetic on the scalar
// pipe, see the tile loop) needs 94 to 118 registers with up to 64 channels per chunk: four
// workgroups share a CU; with up to 128 channels it needs 167, three per CU (the LONG variant of
// that one would spill: two).  The others need up to 256 registers, which leaves room for two.
template <int NDIM, int V, int NCB, int WOUT, bool LONG> constexpr int resident_per_cu()
{
    return (NDIM == 3 && V == 1 && WOUT == 1) ? (NCB <= 4 ? 4 : (LONG ? 2 : 3)) : 2;
}

// Register sets of the channel loop's load pipeline: the loads of stage s + NSETS - 1 are
// issued before the arithmetic of stage s.  A stage is short (a few hundred cycles of
// arithmetic on 2 to 4 KB per wave), so with one stage of lead a wave has at most two stages
// in flight, which at the memory latency under load is not enough to fill the memory
// system; a set costs 8 (3D) to 16 (2D, four voxels per lane) registers.  Four sets where
// they fit without costing a resident workgroup.
template <int NDIM, int V, int NCB, int WOUT, bool LONG> constexpr int pipeline_sets()
{
    return MSD_PIPELINE_SETS_EXPR;
}

// LONG: the variant for what the plain kernel's 32-bit lane offsets and whole-row teams do
// not reach.  The first channel of each block of 16 moves into the uniform base of the x
// loads (so the stack may be of any size and its rows need not be aligned or whole groups of four
// voxels), and rows longer than a workgroup covers are cut into segments, staged with a halo of
// `dil` values on either side.  It is a separate
// instance because even its few extra scalar instructions per stage cost the plain one 1-4 %.
// BIG (LONG instances only): the 64-bit channel bases and the loads from any address; without it
// a LONG instance only cuts rows into segments and addresses like the plain one (whole groups of
// four voxels, stacks below 2^30 values), which saves a fifth of a stage's instructions.
// KONLY: the weight and bias gradients alone (no grad_input update: no weights, no loads or
// stores of grad_input); what is left is the gather, the A tile and a stream over x on the
// matrix cores.  The dense block uses it for two 3D layers per pass, beside a chain of
// backward_x launches on another stream.
template <int NDIM, int V, int NCB, int WOUT, bool LONG, bool BIG = LONG, bool KONLY = false>
__global__ __launch_bounds__(kThreads, (resident_per_cu<NDIM, V, NCB, WOUT, LONG>()))
void bwd_rows_fused(const Args a_, const float *__restrict__ gyp, const float *__restrict__ xp,
                    float *__restrict__ gxp, const float *__restrict__ actp, const float *__restrict__ kw,
                    const float *__restrict__ kw1, const float *__restrict__ kw2, float *__restrict__ part)
{
    // the pointers are separate arguments so that they can carry __restrict__: the weights
    // are then known not to change under the stores to grad_input and stay scalar loads
    extern __shared__ float lds[];
    constexpr int K = Taps<NDIM>::K, NPQ = RowTaps<NDIM>::NPQ;
    constexpr int KR = WOUT * K;                  // rows of the A tile: (output channel, tap)
    constexpr int TG = (KR + 15) / 16;            // groups of 16 such rows
    // 16-voxel MFMA groups per pipeline stage, by measurement: 32 voxels in 2D with four voxels
    // per lane, 16 voxels in 3D up to 64 channels per chunk (these instances then fit the
    // registers of three workgroups per CU without spills), 64 voxels with two voxels per lane
    // (32 with three output channels: the pipeline buffers of 64 would push the accumulators of
    // 128 channels out of the registers)
    constexpr int NSS = V == 1 ? (NCB <= 4 ? 1 : 2) : (V == 4 || WOUT == 3 ? 2 : 4);
    constexpr int H = 4 * V / NSS;                // stages per block of 16 channels (even)
    constexpr int NCS = kChanBlock / H;           // grad_input channels per stage
    constexpr int NSETS = pipeline_sets<NDIM, V, NCB, WOUT, LONG>();   // register sets of the load pipeline
    // 16-voxel stages (one voxel per lane): the x loads of a stage take 64 bytes per channel, half
    // a cache line, and by the time the next stage asks for the other half the line has left the
    // 32 KB vector cache again, so every line of x crosses from the L2 twice; the vector cache's
    // outstanding misses are what bounds the kernel.  XPAIR: x is requested for two stages at a
    // time (both halves of a line together), the rest of the stage (grad_input channels,
    // arithmetic) stays at 16 voxels.
    constexpr bool XPAIR = NDIM == 3 && V == 1 && NSS == 1 && !LONG && MSD_XPAIR;
    static_assert(!XPAIR || (H == 4 && NSETS == 2), "a block is two pairs of stages");
    static_assert(H % NSETS == 0 && NSETS >= 2, "the stages of a block rotate through the register sets");
    constexpr int ASTRIDE = ATile<NDIM, V, WOUT>::kStride;
    // 2D: waves away from the row ends take their x-taps without the mirror arithmetic (3D rows
    // are short: every wave touches an end)
    constexpr bool INNER_PATH = NDIM == 2 && MSD_INNER_PATH;
    const Args &a = a_;
    const Geom &g = a.g;
    const RowTeams &rt = a.rt;
    const int tid = threadIdx.x;
    const int nwaves = blockDim.x / kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), wl = tid % kWave;
    const int mk = wl / 16, mj = wl % 16;         // MFMA k (voxel group) and i/j (tap or channel) of this lane
    // a row team is whole waves (fits()), so the team and everything derived from its row
    // (the source rows of the gather, their clamps and addresses) is wave-uniform: computed
    // from the wave number, it stays in scalar registers and on the scalar pipe
    // (2D keeps the per-lane form: there the scalar registers are the scarcer ones)
    const int team = NDIM == 3 ? (wave * kWave) / rt.lpr : tid / rt.lpr;
    const int lane = tid - team * rt.lpr;
    // segments (rt.segs > 1): a tile is one segment of one row
    constexpr bool SEG = LONG;
    const bool segmented = SEG && a.sg.segs > 1;  // uniform
    const int rs = V * rt.lpr + (SEG ? a.sg.halo : 0);   // floats per staged row
    float *S = lds + (size_t)team * WOUT * NPQ * rs;
    // ALIAS: the waves' tiles lie over the staged rows (the rows are dead once gathered), which
    // takes a workgroup-wide barrier more per tile and brings the instance within the LDS of
    // two workgroups per CU
    constexpr bool ALIAS = tiles_over_staging<NDIM, V, WOUT>();
    float *AT = lds + (ALIAS ? 0 : (size_t)rt.rpw * WOUT * NPQ * rs) + (size_t)wave * ATile<NDIM, V, WOUT>::kFloats;
    if constexpr (!ALIAS)
        for (int i = wl; i < ASTRIDE; i += kWave) AT[KR * ASTRIDE + i] = 0.f;

    const int c0 = blockIdx.z * NCB * kChanBlock;
    const int c_end = min(g.C, c0 + NCB * kChanBlock);   // channels of this chunk end here
    const int cx_end = c_end;
    const int ncb = (c_end - c0 + kChanBlock - 1) / kChanBlock;
    // The bias gradient is the sum of the centre tap over all voxels: every lane adds up its
    // own voxels (chunk 0 only) and the workgroup reduces them at the end.  A virtual input
    // channel of ones on the matrix cores would do it too, but costs a whole block of 16
    // channels more whenever C is a multiple of 16.
    const bool sum_bias = a.want_bias && blockIdx.z == 0;
    float bsum[WOUT];
#pragma unroll
    for (int co = 0; co < WOUT; co++) bsum[co] = 0.f;

    mfma4 D[NCB][TG];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++)
#pragma unroll
        for (int tg = 0; tg < TG; tg++) D[cb][tg] = mfma4{0.f, 0.f, 0.f, 0.f};

    const int lb = block_for_xcd(blockIdx.x, gridDim.x, a.remap);
    const int x0_row = lane * V;
    const int xc_row = min(x0_row, g.W - V);
    const int kx_row = (lane - wl) * V + 4 * mk;  // first voxel of this lane's MFMA groups, + 16 s
    int arow[TG];                                 // this lane's row of the A tile (the zero row past K taps)
#pragma unroll
    for (int tg = 0; tg < TG; tg++) arow[tg] = min(tg * 16 + mj, KR) * ASTRIDE + 4 * mk;

    // Position of the lane's row: divisions here, once; from tile to tile it advances by
    // additions and compares (Args::step).
    int grp = a.group_step == 1 ? lb * a.tiles_per_wg : lb;
    int seg = 0, rg = grp;                                    // uniform: segment of the row, row group
    if constexpr (SEG) {
        seg = grp % a.sg.segs;
        rg = grp / a.sg.segs;
    }
    int gi = rg % a.ngroups, b = rg / a.ngroups;              // uniform: group within the image, batch index
    int row = gi * rt.rpw + team;
    // 3D: (y0, z0) is the first row of the group; 2D: a row is its own y
    int y0 = NDIM == 3 ? (gi * rt.rpw) % g.H : 0, z0 = NDIM == 3 ? (gi * rt.rpw) / g.H : 0;
    int y = NDIM == 3 ? row % g.H : row, z = NDIM == 3 ? row / g.H : 0;

    // The kernel's arguments are the first thing in the argument block.  The 3D instances read
    // them again from there for every tile (scalar loads) instead of keeping them over the
    // channel loop, which has the scalar registers full of weights: kept, they are spilled to
    // lanes of a vector register, every use costs a vector instruction, and the register
    // allocation around them grows (3D, up to 32 channels per chunk: 142-150 -> 108-116 VGPRs,
    // which is what lets a fourth workgroup share the CU).  The 2D instances with two output
    // channels gain 1 % (245 -> 220 VGPRs at most); those with one are 2 % slower that way.
    // One step of the workgroup's walk: from the tile at (grp, seg, gi, b, y0, z0, row, y, z) to its next one.
    auto advance = [&](const Args &a, int &grp, int &seg, int &gi, int &b, int &y0, int &z0, int &row, int &y, int &z) {
        const Geom &g = a.g;
        const RowTeams &rt = a.rt;
        grp += a.group_step;
        int carry = 0;
        if constexpr (SEG) {
            seg += a.step.seg;
            if (seg >= a.sg.segs) {
                seg -= a.sg.segs;
                carry = 1;
            }
        }
        gi += a.step.gi + carry;
        b += a.step.b;
        if constexpr (NDIM == 3) {
            y0 += a.step.y + (carry ? a.step.carry_y : 0);
            z0 += a.step.z + (carry ? a.step.carry_z : 0);
        }
        if (gi >= a.ngroups) {                    // into the next batch item
            gi -= a.ngroups;
            b++;
            if constexpr (NDIM == 3) {
                y0 -= a.step.wrap_y;
                z0 -= a.step.wrap_z;
            }
        }
        row = gi * rt.rpw + team;
        if constexpr (NDIM == 3) {
            while (y0 >= g.H) {
                y0 -= g.H;
                z0++;
            }
            while (y0 < 0) {
                y0 += g.H;
                z0--;
            }
            y = y0 + team;
            z = z0;
            while (y >= g.H) {
                y -= g.H;
                z++;
            }
        } else {
            y = row;
        }
    };
    // KONLY: the first source rows of the tile to come (msd_rows.h: request_source_rows)
    float pre[KONLY ? WOUT : 1][KONLY ? NPQ : 1][V];
    if constexpr (KONLY) {
        if (grp < a.total_groups) {
            const bool ok0 = row < rt.nrows;
            const View<const float> gyv{gyp, a.gy.sb, a.gy.sc, a.gy.sz, a.gy.sy, 1};
            request_source_rows<NDIM, WOUT, V>(g, gyv, b, ok0 ? z : g.D - 1, ok0 ? y : g.H - 1, lane, pre, a.up);
        }
    }
    constexpr bool RELOAD = NDIM == 3 || WOUT == 2;
    typedef const __attribute__((address_space(4))) int *kernarg_words_t;
    kernarg_words_t kernarg = (kernarg_words_t)__builtin_amdgcn_kernarg_segment_ptr();
    for (int ti = 0; ti < a_.tiles_per_wg; ti++) {
        Args again;
        if constexpr (RELOAD) {
            static_assert(sizeof(Args) % sizeof(int) == 0, "Args is made of ints");
            asm volatile("" : "+s"(kernarg));     // a new address as far as the compiler knows: loaded again
            int *dst = reinterpret_cast<int *>(&again);
#pragma unroll
            for (int i = 0; i < (int)(sizeof(Args) / sizeof(int)); i++) dst[i] = kernarg[i];
        }
        const Args &a = [&]() -> const Args & {
            if constexpr (RELOAD) return again; else return a_;
        }();
        const Geom &g = a.g;
        const RowTeams &rt = a.rt;
        if (grp >= a.total_groups) break;         // uniform over the workgroup
        int xsc = a.x.sc, gsc = a.gx.sc;
        asm volatile("" : "+s"(xsc), "+s"(gsc));  // keeps per-channel addresses from being hoisted out of the loop
        const int xs = SEG ? seg * V * rt.lpr : 0;    // first voxel of the segment
        const int x0 = SEG ? xs + x0_row : x0_row;
        const int xc = SEG ? min(x0, g.W - V) : xc_row;
        const int kx = SEG ? xs + kx_row : kx_row;
        const bool rowok = row < rt.nrows;        // teams past the last row work on it again and store nothing
        const bool act = rowok && x0 < g.W;
        const int zc = rowok ? z : g.D - 1, yc = rowok ? y : g.H - 1;
        // Addresses are a wave-uniform 64-bit base (scalar registers) plus a 32-bit byte offset
        // per lane, the form the memory instructions take directly.  x: the lane's channel is
        // part of the offset (LONG: its channel within the block of 16 only); grad_input and
        // activations: the channel is part of the base.
        const uint64_t xbase = reinterpret_cast<uint64_t>(xp + (int64_t)b * a.x.sb);
        const uint32_t xrow = (uint32_t)(zc * a.x.sz + yc * a.x.sy);
        const uint64_t gbase = reinterpret_cast<uint64_t>(gxp + (int64_t)b * a.gx.sb);
        const uint64_t abase = reinterpret_cast<uint64_t>(actp + (int64_t)b * a.gx.sb);
        uint32_t goff = 4u * (uint32_t)(zc * a.gx.sz + yc * a.gx.sy + xc);
        // uniform base of grad_input channel ci, kept in scalar registers
        // (plain instances: the whole of grad_input is below 2^30 values, xkb_mode(), so the
        // channel's byte offset is a 32-bit product: three scalar instructions instead of seven)
        auto channel_base = [&](uint64_t base, int ci) {
            uint64_t p;
            if constexpr (BIG)
                p = base + (uint64_t)((int64_t)ci * gsc * 4);
            else
                p = base + (uint64_t)((uint32_t)ci * (uint32_t)gsc * 4u);
            asm volatile("" : "+s"(p));
            return p;
        };

        // ---- one pipeline stage of loads: NSS 16-voxel groups of 16 channels of x in the MFMA B
        // layout, and NCS channels of grad_input in the voxel layout.  Clamped, always valid
        // addresses; what does not count is replaced after the load.
        float xs_[NSETS][NSS][4];                 // stage s uses set s % NSETS
        float gs_[NSETS][NCS][V];
        auto load_stage = [&](int cb, int h, float (&kk)[NSS][4], float (&gg)[NCS][V]) {
            // (redefining the lane offset keeps its widening to 64 bits next to the loads, where
            // it is free; hoisted out of the loop it would make every address a vector addition)
            asm volatile("" : "+v"(goff));
            if constexpr (BIG) {
                const int cb0 = c0 + cb * kChanBlock;
                const uint64_t xb = xbase + (uint64_t)(uint32_t)cb0 * (uint32_t)(4 * xsc);
                const uint32_t xch = (uint32_t)min(mj, g.C - 1 - cb0) * (uint32_t)xsc + xrow;
#pragma unroll
                for (int j = 0; j < NSS; j++)
                    load_global_vec4_unaligned(xb, 4u * (xch + (uint32_t)min(kx + 16 * (h * NSS + j), g.W - 4)),
                                               kk[j]);
            } else {
                const uint32_t xch = (uint32_t)min(c0 + cb * kChanBlock + mj, g.C - 1) * (uint32_t)xsc + xrow;
#pragma unroll
                for (int j = 0; j < NSS; j++)
                    load_global_vec<4>(xbase, 4u * (xch + (uint32_t)min(kx + 16 * (h * NSS + j), g.W - 4)), kk[j]);
            }
            if constexpr (!KONLY) {
#pragma unroll
                for (int j = 0; j < NCS; j++) {
                    const int ci = max(min(c0 + cb * kChanBlock + h * NCS + j, cx_end - 1), 0);
                    load_global_vec<V>(channel_base(gbase, ci), goff, gg[j]);
                }
            }
        };
        // XPAIR: x of the pair of 16-voxel groups 2 * pair, 2 * pair + 1 (one cache line per channel) ...
        auto load_x2 = [&](int cb, int pair, float (&kk)[2][4]) {
            const uint32_t xch = (uint32_t)min(c0 + cb * kChanBlock + mj, g.C - 1) * (uint32_t)xsc + xrow;
#pragma unroll
            for (int j = 0; j < 2; j++)
                load_global_vec<4>(xbase, 4u * (xch + (uint32_t)min(kx + 16 * (2 * pair + j), g.W - 4)), kk[j]);
        };
        // ... and the grad_input channels of stage h
        auto load_g = [&](int cb, int h, float (&gg)[NCS][V]) {
            asm volatile("" : "+v"(goff));
#pragma unroll
            for (int j = 0; j < NCS; j++) {
                const int ci = max(min(c0 + cb * kChanBlock + h * NCS + j, cx_end - 1), 0);
                load_global_vec<V>(channel_base(gbase, ci), goff, gg[j]);
            }
        };
        float xpa[2][4], xpb[2][4];               // XPAIR: the two pairs of a block alternate
        // block of 16 channels that stage `s` of the walk belongs to
        auto block_of = [&](int s) { return g.reverse ? ncb - 1 - s / H : s / H; };
        // issued ahead of the gather so the latencies overlap (a tile has at least H >= NSETS stages)
        // KONLY: a ring of four pairs of 16-voxel groups, each requested three pairs ahead of its use
        // (two waves per SIMD and nothing but matrix instructions between request and use)
        float xring[KONLY ? 4 : 1][2][4];
        const int npairs = 2 * ncb;
        auto pair_block = [&](int p) {
            const int blk = min(p, npairs - 1) / 2;
            return g.reverse ? ncb - 1 - blk : blk;
        };
        if constexpr (KONLY) {
#pragma unroll
            for (int q = 0; q < 3; q++) load_x2(pair_block(q), min(q, npairs - 1) % 2, xring[q]);
        } else if constexpr (XPAIR) {
            load_x2(block_of(0), 0, xpa);
            load_g(block_of(0), 0, gs_[0]);
        } else {
#pragma unroll
            for (int q = 0; q < NSETS - 1; q++) load_stage(block_of(q), q % H, xs_[q], gs_[q]);
        }

        // ---- A operands, voxel layout: tv[co * K + t][i] = A_co[t](voxel x0 + i of the team's row)
        float tv[KR][V];
        {
            const View<const float> none{nullptr, 0, 0, 0, 0, 0};
            const View<const float> gyv{gyp, a.gy.sb, a.gy.sc, a.gy.sz, a.gy.sy, 1};
            float own[WOUT][NPQ][V];
            if constexpr (KONLY) {
                // the rows were asked for during the tile before (before the loop for the first)
                finish_source_rows<NDIM, WOUT, V>(g, rt, gyv, b, zc, yc, lane, act, S, pre, own, a.up);
            } else if (segmented) {
                if constexpr (SEG)
                    stage_source_segment<NDIM, WOUT, V>(g, rt, a.sg, gyv, b, zc, yc, xs, lane, rowok, S, own, a.up);
            } else {
                stage_source_rows<NDIM, false, WOUT, V>(g, rt, none, gyv, b, zc, yc, lane, act, S, own, a.up);
            }
            // the voxels of this wave: [xw, xw + 64 V) (uniform)
            const int xw = __builtin_amdgcn_readfirstlane(x0);
            // per voxel: all LDS reads first, so that their latencies overlap, then the sums
#pragma unroll
            for (int i = 0; i < V; i++)
#pragma unroll
                for (int co = 0; co < WOUT; co++) {
                    // (the upper output channels may have dilations of their own, and with them their own x-taps)
                    const int dil = dilation_of(g, a.up, co);
                    if (INNER_PATH && xw >= dil && xw + kWave * V + dil <= g.W) {
                        // no lane of the wave is within `dil` of a row end: both x-taps of every
                        // voxel lie inside the row (no mirrored source, nothing to mask): two LDS
                        // reads per staged row instead of four
                        auto at = [&](int p) {    // LDS position of the row's voxel p
                            const int j = p - xs, segw = V * rt.lpr;
                            if (!segmented) return staged_index<V>(p, rt.lpr);
                            return j < 0 ? segw + (j + dil) : (j >= segw ? segw + dil + (j - segw) : staged_index<V>(j, rt.lpr));
                        };
                        const int ihi = at(x0 + i + dil), ilo = at(x0 + i - dil);
                        float rb[NPQ][2];
#pragma unroll
                        for (int pq = 0; pq < NPQ; pq++) {
                            const float *srow = S + (size_t)(co * NPQ + pq) * rs;
                            rb[pq][0] = srow[ihi];
                            rb[pq][1] = srow[ilo];
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int pq = 0; pq < NPQ; pq++) {
                            const int r = co * NPQ + pq;
                            tv[r * 3 + 0][i] = rb[pq][0];
                            tv[r * 3 + 1][i] = own[co][pq][i];
                            tv[r * 3 + 2][i] = rb[pq][1];
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        continue;
                    }
                    const SideTaps<V> side = segmented ? SideTaps<V>(x0 + i, g.W, dil, rt.lpr, xs, V * rt.lpr)
                                                       : SideTaps<V>(min(x0 + i, g.W - 1), g.W, dil, rt.lpr);
                    float ra[NPQ][4];
#pragma unroll
                    for (int pq = 0; pq < NPQ; pq++) {
                        const float *srow = S + (size_t)(co * NPQ + pq) * rs;
                        ra[pq][0] = srow[side.i0a];
                        ra[pq][1] = srow[side.i0b];
                        ra[pq][2] = srow[side.i2a];
                        ra[pq][3] = srow[side.i2b];
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int pq = 0; pq < NPQ; pq++) {
                        const int r = co * NPQ + pq;   // staged row; its three taps are rows 3 r .. 3 r + 2 of tv
                        tv[r * 3 + 0][i] = (side.m0a ? ra[pq][0] : 0.f) + (side.m0b ? ra[pq][1] : 0.f);
                        tv[r * 3 + 1][i] = own[co][pq][i];
                        tv[r * 3 + 2][i] = (side.m2a ? ra[pq][2] : 0.f) + (side.m2b ? ra[pq][3] : 0.f);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            __syncthreads();                      // the staged rows may be overwritten from here on
            if constexpr (ALIAS)
                for (int i = wl; i < ASTRIDE; i += kWave) AT[KR * ASTRIDE + i] = 0.f;
            // the wave's [row][voxel] tile; lanes past the image row hold finite values that meet zeros of x
#pragma unroll
            for (int t = 0; t < KR; t++) store_vec<V>(AT + t * ASTRIDE + wl * V, tv[t]);
            if (sum_bias && act) {
#pragma unroll
                for (int co = 0; co < WOUT; co++)
#pragma unroll
                    for (int i = 0; i < V; i++) bsum[co] += tv[co * K + K / 2][i];
            }
        }
        if constexpr (KONLY) {
            // the next tile's source rows, in flight during this tile's channel loop
            int ngrp = grp, nseg = seg, ngi = gi, nb = b, ny0 = y0, nz0 = z0, nrow = row, ny = y, nz = z;
            advance(a, ngrp, nseg, ngi, nb, ny0, nz0, nrow, ny, nz);
            if (ti + 1 < a_.tiles_per_wg && ngrp < a.total_groups) {
                const bool nok = nrow < rt.nrows;
                const View<const float> gyv{gyp, a.gy.sb, a.gy.sc, a.gy.sz, a.gy.sy, 1};
                request_source_rows<NDIM, WOUT, V>(g, gyv, nb, nok ? nz : g.D - 1, nok ? ny : g.H - 1, lane, pre, a.up);
            }
        }
        // the tile is private to the wave and LDS executes a wave's accesses in order: only
        // the compiler has to be kept from reordering them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // Accumulation chains per tap group: two where there is one group (dependent matrix
        // instructions would wait for each other), one where the groups already alternate.
        constexpr int NCH = TG >= 2 ? 1 : 2;
        mfma4 acc[TG][NCH];
        // weight gradient of one stage: 4 * NSS * TG matrix instructions
        auto stage_k = [&](int cb, int h, float (&kk)[NSS][4]) {
            const int chl = c0 + cb * kChanBlock + mj;
            const bool chok = chl < g.C;
#pragma unroll
            for (int j = 0; j < NSS; j++) {
                const int s = h * NSS + j;
                const bool vok = rowok && kx + 16 * s < g.W;
                const bool keep = vok && chok;
                if constexpr (BIG) {
                    // rows need not be whole groups of four voxels here: the last group of a row
                    // was loaded from W - 4 (inside the row), `shift` voxels early; move its
                    // values down and fill with zeros
                    // (selects, no branch: nothing in the channel loop depends on the lane)
                    const int shift = kx + 16 * s - (g.W - 4);
                    const float r[8] = {kk[j][0], kk[j][1], kk[j][2], kk[j][3], 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        kk[j][e] = shift <= 0 ? r[e]
                                              : (shift == 1 ? r[e + 1]
                                                            : (shift == 2 ? r[e + 2] : (shift == 3 ? r[e + 3] : 0.f)));
                }
                f32x4 av[TG];
#pragma unroll
                for (int tg = 0; tg < TG; tg++) av[tg] = *reinterpret_cast<const f32x4 *>(AT + arow[tg] + 16 * s);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float bv = keep ? kk[j][e] : 0.f;
#pragma unroll
                    for (int tg = 0; tg < TG; tg++)
                        acc[tg][e % NCH] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(av[tg][e], bv, acc[tg][e % NCH], 0, 0, 0);
                }
            }
        };
        // grad_input of one channel: WOUT * K * V fused multiply-adds with the channel's weights
        // (wave-uniform: scalar loads into scalar registers), then the store
        auto load_weights = [&](int ci, float (&w)[KR]) {
#pragma unroll
            for (int co = 0; co < WOUT; co++) {
                const float *kc = (co == 0 ? kw : (co == 1 ? kw1 : kw2)) + (uint32_t)(ci * K);
#pragma unroll
                for (int t = 0; t < K; t++) w[co * K + t] = kc[t];
            }
        };
        // `prefetch`: the weights of the next channel are requested right after the first use
        // of this channel's (scalar loads return in any order, so only a wait for all of them
        // exists: the request must follow that wait to have the rest of the arithmetic to land in)
        auto update_channel = [&](int ci, float (&gv)[V], const float (&w)[KR], auto prefetch, float (&wn)[KR],
                                  bool masked) {
            float sum[V];
#pragma unroll
            for (int i = 0; i < V; i++) sum[i] = w[0] * tv[0][i];
            __builtin_amdgcn_sched_barrier(0);
            if (decltype(prefetch)::value) load_weights(ci + 1, wn);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 1; t < KR; t++)
#pragma unroll
                for (int i = 0; i < V; i++) sum[i] += w[t] * tv[t][i];
#pragma unroll
            for (int i = 0; i < V; i++) gv[i] += sum[i];
            if (masked) {
                // an output of the layer below: its gradient is complete with this update, so its
                // ReLU mask is applied on the way out
                float m[V];
                load_global_vec<V>(channel_base(abase, ci), goff, m);
#pragma unroll
                for (int i = 0; i < V; i++) gv[i] = 0.f < m[i] ? gv[i] : 0.f;
            }
            store_global_vec<V>(channel_base(gbase, ci), goff, gv);
        };
        // grad_input of one stage: up to NCS channels.  Lanes past the row sit the whole stage
        // out, so that the channels form one straight run of code; the stage that holds masked
        // channels or the end of the channel range goes channel by channel instead.
        auto stage_x = [&](int cb, int h, float (&gg)[NCS][V]) {
            const int cj0 = c0 + cb * kChanBlock + h * NCS;
            if (!act) return;
            asm volatile("" : "+v"(goff));        // as in load_stage: the stores take base + lane offset directly
            float w[2][KR];
            if (cj0 + NCS <= min(cx_end, a.mask_from)) {   // uniform
                load_weights(cj0, w[0]);
#pragma unroll
                for (int j = 0; j < NCS; j++) {
                    if (j + 1 < NCS)
                        update_channel(cj0 + j, gg[j], w[j & 1], std::true_type{}, w[(j + 1) & 1], false);
                    else
                        update_channel(cj0 + j, gg[j], w[j & 1], std::false_type{}, w[(j + 1) & 1], false);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NCS; j++)
                    if (cj0 + j < cx_end) {
                        load_weights(cj0 + j, w[0]);
                        update_channel(cj0 + j, gg[j], w[0], std::false_type{}, w[1], cj0 + j >= a.mask_from);
                    }
            }
        };

        // ---- channel loop: blocks of 16 channels, H stages each, NSETS stages per iteration (all of
        // one block); the loads of stage s + NSETS - 1 are issued before the arithmetic of stage s
        const int nst = ncb * H;                  // a multiple of NSETS
        if constexpr (KONLY) {
            // x alone: four pairs (two blocks of 16 channels) per iteration of the loop
            static_assert(XPAIR, "the weight-gradient-only instances are the 3D ones with one voxel per lane");
#pragma unroll 1
            for (int p0 = 0; p0 < npairs; p0 += 4) {
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int p = p0 + u;
                    // (past the last pair the last one is asked for again: never used, a cache hit)
                    load_x2(pair_block(p + 3), min(p + 3, npairs - 1) % 2, xring[(u + 3) % 4]);
                    if (p < npairs) {             // uniform
                        const int cb = pair_block(p);
                        if (u % 2 == 0) {
#pragma unroll
                            for (int tg = 0; tg < TG; tg++)
#pragma unroll
                                for (int c = 0; c < NCH; c++) acc[tg][c] = mfma4{0.f, 0.f, 0.f, 0.f};
                        }
                        stage_k(cb, 2 * (u % 2), reinterpret_cast<float (&)[NSS][4]>(xring[u][0]));
                        stage_k(cb, 2 * (u % 2) + 1, reinterpret_cast<float (&)[NSS][4]>(xring[u][1]));
                        if (u % 2 == 1) {
#pragma unroll
                            for (int q = 0; q < NCB; q++)
                                if (q == cb) {
#pragma unroll
                                    for (int tg = 0; tg < TG; tg++)
#pragma unroll
                                        for (int c = 0; c < NCH; c++) D[q][tg] += acc[tg][c];
                                }
                        }
                    }
                }
            }
        } else if constexpr (XPAIR) {
            // one block of 16 channels (four stages) per iteration.  Every load is issued a stage
            // or more ahead of its use and none sits behind a test (loads retire in order, and the
            // compiler sizes each wait for the path with the fewest loads behind the one it needs):
            // past the last block the loads ask for lines of this block again.
#pragma unroll 1
            for (int blk = 0; blk < ncb; blk++) {
                const int cb = g.reverse ? ncb - 1 - blk : blk;
                const bool more = blk + 1 < ncb;
                const int cbn = more ? (g.reverse ? cb - 1 : cb + 1) : cb;
#pragma unroll
                for (int tg = 0; tg < TG; tg++)
#pragma unroll
                    for (int c = 0; c < NCH; c++) acc[tg][c] = mfma4{0.f, 0.f, 0.f, 0.f};
                load_g(cb, 1, gs_[1]);
                load_x2(cb, 1, xpb);
                stage_k(cb, 0, reinterpret_cast<float (&)[NSS][4]>(xpa[0]));
                stage_x(cb, 0, gs_[0]);
                load_g(cb, 2, gs_[0]);
                stage_k(cb, 1, reinterpret_cast<float (&)[NSS][4]>(xpa[1]));
                stage_x(cb, 1, gs_[1]);
                load_g(cb, 3, gs_[1]);
                load_x2(cbn, more ? 0 : 1, xpa);
                stage_k(cb, 2, reinterpret_cast<float (&)[NSS][4]>(xpb[0]));
                stage_x(cb, 2, gs_[0]);
                load_g(cbn, more ? 0 : 3, gs_[0]);
                stage_k(cb, 3, reinterpret_cast<float (&)[NSS][4]>(xpb[1]));
                stage_x(cb, 3, gs_[1]);
#pragma unroll
                for (int q = 0; q < NCB; q++)
                    if (q == cb) {
#pragma unroll
                        for (int tg = 0; tg < TG; tg++)
#pragma unroll
                            for (int c = 0; c < NCH; c++) D[q][tg] += acc[tg][c];
                    }
            }
        } else
#pragma unroll 1
        for (int st = 0; st < nst; st += NSETS) {
            const int cb = block_of(st);
#pragma unroll
            for (int tg = 0; tg < TG; tg++)
#pragma unroll
                for (int c = 0; c < NCH; c++) acc[tg][c] = mfma4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < NSETS; u++) {
                const int h = st % H + u;
                constexpr int kLead = NSETS - 1;
                float (&kn)[NSS][4] = xs_[(u + kLead) % NSETS];
                float (&gn)[NCS][V] = gs_[(u + kLead) % NSETS];
                // 2D: no test around these loads.  Loads and stores retire through one in-order
                // counter and the compiler derives each wait from what may be pending on any path,
                // so a load that may be skipped turns the wait in front of the next matrix
                // instructions into one for these loads themselves.  Past the last stage a stage
                // of this tile is loaded again instead (cache hits, never used).  Measured with two
                // sets: 2 % faster in 2D, 2 % slower in 3D (fewer, longer iterations per tile),
                // which keeps the test.
                if constexpr (NDIM == 2) {
                    const int sn = min(st + u + kLead, nst - 1);
                    load_stage(block_of(sn), sn % H, kn, gn);
                } else {
                    const int sn = st + u + kLead;
                    if (sn < nst) load_stage(block_of(sn), sn % H, kn, gn);
                }
                stage_k(cb, h, xs_[u]);
                stage_x(cb, h, gs_[u]);
            }
            // D is indexed statically: pick the block with a chain of uniform branches
#pragma unroll
            for (int q = 0; q < NCB; q++)
                if (q == cb) {
#pragma unroll
                    for (int tg = 0; tg < TG; tg++)
#pragma unroll
                        for (int c = 0; c < NCH; c++) D[q][tg] += acc[tg][c];
                }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if constexpr (ALIAS) __syncthreads();     // the next tile's staged rows overwrite every wave's tile
        // next tile (all of this is uniform)
        advance(a, grp, seg, gi, b, y0, z0, row, y, z);
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
    // partial sums are stored column-major, part[column][workgroup], so that the
    // second pass reads each column as one contiguous run
    float *pcol = part + blockIdx.x;
    for (int idx = tid; idx < PER_WAVE; idx += blockDim.x) {
        const int l = idx % kWave, v = (idx / kWave) % 4, tg = (idx / (4 * kWave)) % TG, cb = idx / (4 * kWave * TG);
        const int r = tg * 16 + 4 * (l / 16) + v;     // row of the A tile: (output channel, tap)
        const int ch = c0 + cb * kChanBlock + l % 16;
        if (r >= KR || ch >= c_end) continue;
        const int co = r / K, tap = r % K;
        float s = 0.f;
        for (int w = 0; w < nwaves; w++) s += red[w * PER_WAVE + idx];
        pcol[(((int64_t)co * g.C + ch) * K + tap) * kMaxPartialRows] = s;
    }
    if (sum_bias) {                               // uniform over the workgroup
        // lanes of a wave by a fixed shuffle tree, then the waves in order
        __syncthreads();
#pragma unroll
        for (int co = 0; co < WOUT; co++) {
            float s = bsum[co];
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_down(s, off, kWave);
            if (wl == 0) red[wave * WOUT + co] = s;
        }
        __syncthreads();
        if (tid < WOUT) {
            float s = 0.f;
            for (int w = 0; w < nwaves; w++) s += red[w * WOUT + tid];
            pcol[((int64_t)WOUT * g.C * K + tid) * kMaxPartialRows] = s;
        }
    }
}

template <int NDIM, int V, int NCB, int WOUT>
size_t lds_bytes(const RowTeams &rt, const RowSegments &sg)
{
    constexpr int TG = (WOUT * Taps<NDIM>::K + 15) / 16;
    const size_t staged = (size_t)rt.rpw * WOUT * RowTaps<NDIM>::NPQ * (V * rt.lpr + sg.halo) * 4;
    const size_t tiles = (size_t)kWaves * ATile<NDIM, V, WOUT>::kFloats * 4;
    const size_t main_loop = tiles_over_staging<NDIM, V, WOUT>() ? std::max(staged, tiles) : staged + tiles;
    const size_t epilogue = (size_t)kWaves * NCB * TG * 4 * kWave * 4;
    return std::max(main_loop, epilogue);
}

constexpr size_t kMaxLdsBytes = 64 * 1024;
// what the instances with tiles over the staged rows ask for (an opt-in per kernel): two such
// workgroups fill the 160 KB of a CU
constexpr size_t kMaxLdsBytesAsked = 80 * 1024;

// Strides and in-plane offsets fit the kernel's 32-bit arithmetic.
template <typename T>
inline bool small_strides(const Geom &g, const View<T> &v)
{
    const int64_t lim = (int64_t)1 << 30;
    if (v.sb >= lim * 2 || v.sc >= lim * 2 || v.sz >= lim || v.sy >= lim) return false;
    return (int64_t)(g.D - 1) * v.sz + (int64_t)(g.H - 1) * v.sy + g.W < lim;
}

// Usable with V voxels per lane: whole waves per row, rows fit a 256-lane workgroup,
// 16-byte accesses to x and V-wide ones to the other tensors aligned.
template <int NDIM>
bool fits(const Geom &g, int V, const View<const float> &gy, const View<const float> &x, const View<float> &gx,
          bool lng)
{
    RowTeams rt;
    RowSegments sg;
    // the plain kernel loads x in aligned groups of four voxels; the LONG one from any address
    if (lng ? g.W < 4 : (g.W % 4 != 0 || !rows_aligned(x, g.W, 4))) return false;
    sg = RowSegments{1, 0};
    if (!make_row_teams(g, V, &rt, lng ? &sg : nullptr)) return false;
    if (rt.lpr % kWave != 0 || rt.lpr * rt.rpw > kThreads) return false;
    // staged rows + the waves' A tiles within the 64 KB of LDS a workgroup may ask for without
    // opting in to more (3D rows of 512 voxels at two voxels per lane would take 77 KB: such
    // rows are cut into segments by the LONG instances instead)
    const size_t kr = (size_t)g.Wd * Taps<NDIM>::K + 1;
    const size_t staged = (size_t)rt.rpw * g.Wd * RowTaps<NDIM>::NPQ * (V * rt.lpr + sg.halo) * 4;
    const size_t tiles = (size_t)kWaves * kr * (kWave * V + 4) * 4;
    const bool over = (NDIM == 2 && ((V == 4 && g.Wd == 2) || g.Wd == 3)) || (NDIM == 3 && (V == 2 || g.Wd >= 2));   // tiles_over_staging()
    if ((over ? std::max(staged, tiles) : staged + tiles) > (over ? kMaxLdsBytesAsked : kMaxLdsBytes)) return false;
    return rows_aligned(gy, g.W, V) && rows_aligned(gx, g.W, V);
}

template <int NDIM>
int choose_vec(const Geom &g, int vmax, const View<const float> &gy, const View<const float> &x,
               const View<float> &gx, bool lng)
{
    // 3D: one voxel per lane where that covers the row (27 gathered taps per voxel: twice the
    // resident waves, 10 % faster at 128^3); two, with the waves' tiles over the staged rows, for
    // rows of 257 to 512 voxels, which otherwise go in segments (15-20 % slower)
    for (int v = NDIM == 3 ? (lng ? 1 : 2) : 4; v >= 1; v /= 2) {
        if (v > vmax) continue;
        if (fits<NDIM>(g, v, gy, x, gx, lng)) return v;
    }
    return 0;
}

// `group`: the output channels are layers of a dense block (g.dil is then the largest of their
// dilations, which is what the row segments' halo is sized for).
template <int NDIM, int V, int NCB, int WOUT, bool LONG, bool BIG = LONG, bool KONLY = false>
hipError_t launch(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                  const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws, hipStream_t s,
                  ReduceJob *defer, const LayerGroup *group)
{
    constexpr int K = Taps<NDIM>::K;
    Args a;
    a.g = g;
    a.up = UpperDilations{{0, 0}};
    if (group) {
        if (WOUT != group->n || WOUT < 2 || WOUT > kMaxLayerGroup) return hipErrorInvalidValue;
        a.g.dil = group->dil[0];
        for (int co = 1; co < WOUT; co++) a.up.d[co - 1] = group->dil[co];
    }
    a.sg = RowSegments{1, 0};
    make_row_teams(g, V, &a.rt, LONG ? &a.sg : nullptr);
    // a deferred reduction brings its own region for the partial sums (defer->part)
    float *part = defer ? const_cast<float *>(defer->part) : ws + backward_k_mask_floats(g);
    a.ngroups = (a.rt.nrows + a.rt.rpw - 1) / a.rt.rpw;
    const int64_t total = (int64_t)a.ngroups * a.sg.segs * g.B;
    a.remap = knob(kKnobXcdRemap, 1);
    // as many workgroups as are resident at once (256 CUs): the grid then runs as one round
    const int64_t max_wgs = std::min<int64_t>(
        std::max(8, knob(kKnobBwdkBlocks, group && group->max_workgroups > 0
                                              ? group->max_workgroups
                                              : 256 * resident_per_cu<NDIM, V, NCB, WOUT, LONG>())),
        kMaxPartialRows);
    a.tiles_per_wg = (int)((total + max_wgs - 1) / max_wgs);
    const int64_t wgs = (total + a.tiles_per_wg - 1) / a.tiles_per_wg;
    const int rows = a.remap ? xcd_grid((int)wgs) : (int)wgs;   // padding workgroups write zero rows
    if (rows > kMaxPartialRows || total > INT32_MAX) return hipErrorInvalidConfiguration;
    a.group_step = 1;
    if (knob(kKnobBwdkInterleave, 1) && total + rows < INT32_MAX) {
        // the workgroups sweep the image together: at any time they work on one window of
        // consecutive rows, every workgroup on every rows-th group
        a.group_step = rows;
        a.tiles_per_wg = (int)((total + rows - 1) / rows);
    }
    a.total_groups = (int)total;
    {
        const int s_rg = a.group_step / a.sg.segs, rows_step = (a.group_step / a.sg.segs % a.ngroups) * a.rt.rpw;
        a.step.seg = a.group_step % a.sg.segs;
        a.step.gi = s_rg % a.ngroups;
        a.step.b = s_rg / a.ngroups;
        a.step.y = rows_step % g.H;
        a.step.z = rows_step / g.H;
        a.step.wrap_y = (a.ngroups * a.rt.rpw) % g.H;
        a.step.wrap_z = (a.ngroups * a.rt.rpw) / g.H;
        a.step.carry_y = a.rt.rpw % g.H;
        a.step.carry_z = a.rt.rpw / g.H;
    }
    a.gy = Plane{(int)gy.sb, (int)gy.sc, (int)gy.sz, (int)gy.sy};
    a.x = Plane{(int)x.sb, (int)x.sc, (int)x.sz, (int)x.sy};
    a.gx = Plane{(int)gx.sb, (int)gx.sc, (int)gx.sz, (int)gx.sy};
    const float *actp = pm.from < g.C ? pm.act.p : x.p;   // only dereferenced for channels >= mask_from
    a.mask_from = pm.from;
    a.want_bias = gb != nullptr;
    const int chunks = (g.C + NCB * kChanBlock - 1) / (NCB * kChanBlock);
    const size_t lds = lds_bytes<NDIM, V, NCB, WOUT>(a.rt, a.sg);
    constexpr bool kAsks = tiles_over_staging<NDIM, V, WOUT>();
    if (lds > (kAsks ? kMaxLdsBytesAsked : kMaxLdsBytes)) return hipErrorInvalidConfiguration;   // excluded by fits()
    if (kAsks && lds > kMaxLdsBytes) {
        // more than 64 KB has to be asked for, once per kernel and device (the attribute stays):
        // later launches, also ones recorded into a graph, go without the call
        static std::atomic<uint64_t> asked{0};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const uint64_t bit = dev >= 0 && dev < 64 ? (uint64_t)1 << dev : 0;
        if (!(asked.load(std::memory_order_acquire) & bit)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&bwd_rows_fused<NDIM, V, NCB, WOUT, LONG, BIG, KONLY>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLdsBytesAsked);
            if (e != hipSuccess) return e;
            asked.fetch_or(bit, std::memory_order_release);
        }
    }
    // the weights of the upper output channels follow those of the first, or are other layers'
    const float *k1 = group ? group->k_up[0] : k + (int64_t)g.C * K;
    const float *k2 = group ? group->k_up[1] : k + (int64_t)2 * g.C * K;
    hipLaunchKernelGGL((bwd_rows_fused<NDIM, V, NCB, WOUT, LONG, BIG, KONLY>), dim3(rows, 1, chunks), dim3(a.rt.lpr * a.rt.rpw), lds, s, a,
                       gy.p, x.p, gx.p, actp, k, k1, k2, part);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t nk = (int64_t)WOUT * g.C * K;
    const int64_t ncols = nk + (a.want_bias ? WOUT : 0);
    // a group's columns: [0, split) of the partial sums go to gk, the next `split` ones to the
    // second layer's weight gradient, the rest to the third's
    // (KONLY pairs run over one channel more than the lower layer has: its columns of that
    // channel are dropped by the reduction)
    const int64_t per_layer = group ? (int64_t)g.C * K : nk;
    const ReduceJob job{part, gk, gb, nk, ncols, rows, {group ? group->gk_up[0] : nullptr, group ? group->gk_up[1] : nullptr},
                        per_layer, group && group->lowest_channels > 0 ? (int64_t)group->lowest_channels * K : per_layer};
    if (defer) {
        *defer = job;
        return hipSuccess;
    }
    if (group) return reduce_columns_batch(&job, 1, s);   // (adds in the same order)
    hipLaunchKernelGGL(bwdk::reduce_columns, dim3((ncols + 3) / 4), dim3(256), 0, s, part, rows, nk, ncols, gk, gb);
    return hipGetLastError();
}

template <int NDIM, int V, int WOUT, bool LONG, bool BIG = LONG>
hipError_t pick_ncb(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                    const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws, hipStream_t s,
                    ReduceJob *defer, const LayerGroup *group)
{
    const int need = (g.C + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch<NDIM, V, 1, WOUT, LONG, BIG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    if (need <= 2) return launch<NDIM, V, 2, WOUT, LONG, BIG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    if (need <= 4) return launch<NDIM, V, 4, WOUT, LONG, BIG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    if constexpr (WOUT == 3) {
        // three output channels: the accumulators of 128 channels spill a few registers, those of 96 do not
        if (need <= 6) return launch<NDIM, V, 6, WOUT, LONG, BIG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
    }
    return launch<NDIM, V, 8, WOUT, LONG, BIG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
}

// Widest vector for two output channels (2D only): twice the gathered values per voxel must
// still fit the registers beside the pipeline buffers.
constexpr int kMaxVecTwoOutputs = 2;
// ... four in the plain kernel, whose tiles lie over the staged rows
constexpr int kMaxVecTwoOutputsPlain = 4;

// Lane offsets into x fit 32 bits: they span the whole stack in the plain kernel, one block
// of 16 channels in the LONG one.  The plain kernel asks the same of grad_input (its channel
// offsets are 32-bit products).
inline bool x_offsets_fit(const Geom &g, const View<const float> &x, bool lng)
{
    const int64_t channels = lng ? kChanBlock : g.C;
    return channels * x.sc + (int64_t)g.D * x.sz + (int64_t)g.H * x.sy + g.W < ((int64_t)1 << 30);
}

enum Mode { kUnsupported = 0, kPlain = 1, kLong = 2 };

// One output channel (2D: one or two), unit x-strides, 32-bit strides, and a vector width
// that fits: with the plain kernel where it reaches, else with the LONG one.
template <int NDIM>
Mode xkb_mode(const Geom &g, const View<const float> &gy, const View<const float> &x, const View<float> &gx)
{
    if (g.Wd != 1 && !(NDIM == 2 && (g.Wd == 2 || g.Wd == 3))) return kUnsupported;
    if (x.sx != 1 || gy.sx != 1 || gx.sx != 1) return kUnsupported;
    if (!small_strides(g, gy) || !small_strides(g, x) || !small_strides(g, gx)) return kUnsupported;
    const int vmax = g.Wd >= 2 ? kMaxVecTwoOutputs : 4;
    const View<const float> gxc{gx.p, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
    if (g.Wd == 3) {
        // three output channels: aligned rows of whole groups of four voxels, two voxels per lane,
        // offsets within 32 bits; nothing else
        if (!x_offsets_fit(g, x, false) || !x_offsets_fit(g, gxc, false)) return kUnsupported;
        if (g.W % 4 == 0 && rows_aligned(x, g.W, 4) && choose_vec<NDIM>(g, kMaxVecTwoOutputs, gy, x, gx, true) == 2)
            return kLong;
        return kUnsupported;
    }
    const int vmax_plain = g.Wd == 2 ? kMaxVecTwoOutputsPlain : 4;
    if (x_offsets_fit(g, x, false) && x_offsets_fit(g, gxc, false) &&
        choose_vec<NDIM>(g, vmax_plain, gy, x, gx, false) != 0)
        return kPlain;
    if (x_offsets_fit(g, x, true) && choose_vec<NDIM>(g, vmax, gy, x, gx, true) != 0) return kLong;
    return kUnsupported;
}

// pm.act, where pm.from < C, must be laid out like gx (same strides and 16-byte phase).
template <int NDIM, bool LONG>
hipError_t xkb_nd(const Geom &g, const View<const float> &gy, const View<const float> &x, const float *k,
                  const View<float> &gx, const PostMask &pm, float *gk, float *gb, float *ws, hipStream_t s,
                  ReduceJob *defer, const LayerGroup *group = nullptr)
{
    // 3D: one voxel per lane keeps the 27 gathered values per voxel and the pipeline buffers in registers
    int vmax = knob(NDIM == 3 ? kKnobBwdkVec3d : kKnobBwdkVec2d, NDIM == 3 ? 1 : 4);
    if (NDIM == 2 && !LONG && knob(kKnobBwdkVec2d, -1) < 0) {
        // Small images: fewer voxels per lane make more tiles (a tile is 256 lanes: one long row or
        // several short ones).  The widest vector that still fills the 512 resident workgroups
        // wins, else the one with the most tiles (256 x 256, 100 channels: 58 -> 39 us).
        int best = 0;
        int64_t best_tiles = 0;
        for (int v = g.Wd == 3 ? kMaxVecTwoOutputs : (g.Wd == 2 ? kMaxVecTwoOutputsPlain : 4); v >= 1; v /= 2) {
            RowTeams rt;
            if (!fits<NDIM>(g, v, gy, x, gx, LONG) || !make_row_teams(g, v, &rt)) continue;
            const int64_t tiles = (int64_t)g.B * ((rt.nrows + rt.rpw - 1) / rt.rpw);
            if (tiles > best_tiles) { best = v; best_tiles = tiles; }
            if (tiles >= 512) break;
        }
        if (best) vmax = best;
    }
    int v = choose_vec<NDIM>(g, vmax, gy, x, gx, LONG);
    if (v == 0) v = choose_vec<NDIM>(g, 4, gy, x, gx, LONG);
    if constexpr (NDIM == 2) {
        if (g.Wd == 3) {
            // three output channels: two voxels per lane in the instance that cuts long rows into
            // segments and is otherwise like the plain one (xkb_mode), also for rows that one
            // workgroup covers (the plain form of it would spill registers)
            if constexpr (LONG) {
                if (choose_vec<2>(g, kMaxVecTwoOutputs, gy, x, gx, true) == 2)
                    return pick_ncb<2, 2, 3, true, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
            }
            return hipErrorInvalidConfiguration;
        }
        if (g.Wd == 2) {
            constexpr int vmax2 = LONG ? kMaxVecTwoOutputs : kMaxVecTwoOutputsPlain;
            v = choose_vec<2>(g, std::min(vmax, vmax2), gy, x, gx, LONG);
            if (v == 0) v = choose_vec<2>(g, vmax2, gy, x, gx, LONG);
            if constexpr (LONG) {
                // rows that are only long (whole groups of four voxels, aligned, offsets within 32
                // bits like the plain kernel asks): segments without the other LONG machinery
                const View<const float> gxc{gx.p, gx.sb, gx.sc, gx.sz, gx.sy, gx.sx};
                const bool segments_only = g.W % 4 == 0 && rows_aligned(x, g.W, 4) && x_offsets_fit(g, x, false) &&
                                           x_offsets_fit(g, gxc, false);
                if (segments_only && vmax >= 4 && choose_vec<2>(g, 4, gy, x, gx, true) == 4)
                    return pick_ncb<2, 4, 2, true, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
                if (segments_only && v == 2)
                    return pick_ncb<2, 2, 2, true, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
                if (segments_only && v == 1)
                    return pick_ncb<2, 1, 2, true, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
            }
            if constexpr (!LONG)
                if (v == 4) return pick_ncb<2, 4, 2, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
            if (v == 2) return pick_ncb<2, 2, 2, LONG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
            if (v == 1) return pick_ncb<2, 1, 2, LONG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, group);
            return hipErrorInvalidConfiguration;
        }
        if (v == 4) return pick_ncb<2, 4, 1, LONG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, nullptr);
    }
    if (g.Wd != 1) return hipErrorInvalidConfiguration;
    if constexpr (NDIM == 2) {
        if (v == 2) return pick_ncb<2, 2, 1, LONG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, nullptr);
    }
    if constexpr (NDIM == 3 && !LONG) {
        if (v == 2) return pick_ncb<3, 2, 1, false>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, nullptr);
    }
    if (v == 1) return pick_ncb<NDIM, 1, 1, LONG>(g, gy, x, k, gx, pm, gk, gb, ws, s, defer, nullptr);
    return hipErrorInvalidConfiguration;
}

// Weight and bias gradients of two 3D layers of a dense block in one pass over the input
// channels of the upper one (plain instances, one voxel per lane, up to 64 channels per chunk
// of the grid): whether the shapes fit, and the launch.
inline bool k_pair_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x)
{
    if (g.ndim != 3 || g.Wd != 2 || x.sx != 1 || gy.sx != 1) return false;
    if (!small_strides(g, gy) || !small_strides(g, x) || !x_offsets_fit(g, x, false)) return false;
    const View<float> none{const_cast<float *>(gy.p), gy.sb, gy.sc, gy.sz, gy.sy, gy.sx};   // (grad_input is not touched)
    return fits<3>(g, 1, gy, x, none, false);
}

inline hipError_t k_pair_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk, float *gb,
                            float *ws, hipStream_t s, ReduceJob *defer, const LayerGroup *group)
{
    const View<float> none{nullptr, 0, 0, 0, 0, 1};
    const PostMask pm{g.C, {nullptr, 0, 0, 0, 0, 0}};
    const int need = (g.C + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch<3, 1, 1, 2, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, defer, group);
    if (need <= 2) return launch<3, 1, 2, 2, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, defer, group);
    return launch<3, 1, 4, 2, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, defer, group);
}

// Weight and bias gradients of one 3D layer of one or two output channels (one dilation) from
// its masked output gradient: the same instances without a group, and those of one output
// channel.
inline bool k_only_supported_3d(const Geom &g, const View<const float> &gy, const View<const float> &x)
{
    if (g.ndim != 3 || g.Wd < 1 || g.Wd > 2 || x.sx != 1 || gy.sx != 1) return false;
    if (!small_strides(g, gy) || !small_strides(g, x) || !x_offsets_fit(g, x, false)) return false;
    const View<float> none{const_cast<float *>(gy.p), gy.sb, gy.sc, gy.sz, gy.sy, gy.sx};   // (grad_input is not touched)
    return fits<3>(g, 1, gy, x, none, false);
}

template <int WOUT>
inline hipError_t k_only_3d_w(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk,
                              float *gb, float *ws, hipStream_t s)
{
    const View<float> none{nullptr, 0, 0, 0, 0, 1};
    const PostMask pm{g.C, {nullptr, 0, 0, 0, 0, 0}};
    const int need = (g.C + kChanBlock - 1) / kChanBlock;
    if (need <= 1) return launch<3, 1, 1, WOUT, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, nullptr, nullptr);
    if (need <= 2) return launch<3, 1, 2, WOUT, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, nullptr, nullptr);
    return launch<3, 1, 4, WOUT, false, false, true>(g, gy, x, nullptr, none, pm, gk, gb, ws, s, nullptr, nullptr);
}

inline hipError_t k_only_3d(const Geom &g, const View<const float> &gy, const View<const float> &x, float *gk, float *gb,
                            float *ws, hipStream_t s)
{
    return g.Wd == 1 ? k_only_3d_w<1>(g, gy, x, gk, gb, ws, s) : k_only_3d_w<2>(g, gy, x, gk, gb, ws, s);
}

}  // namespace bwdxk
}  // namespace msd
