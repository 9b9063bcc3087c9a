// Column reductions of several layers in one launch.
//
// The weight-gradient kernels leave one row of partial sums per workgroup in the workspace,
// part[column][kMaxPartialRows].  A reduction of its own per layer is a 4 microsecond launch
// between two large kernels; the dense block's reverse loop instead keeps the partial sums
// of up to kReduceBatch layers in separate regions and reduces them together.
#include "msd_kernels.h"

namespace msd {
namespace {

struct ReduceBatch {
    ReduceJob job[kReduceBatch];
    int64_t first[kReduceBatch + 1];              // first global column of each job; first[n] = all columns
    int n;
};

// One wave per column, columns numbered through all jobs.  Lane l adds rows l, l + 64, ... in
// order, then the 64 lane sums are added by a fixed shuffle tree: the order of
// bwdk::reduce_columns, so the result is the same whichever of the two ran.
__global__ __launch_bounds__(256) void reduce_columns_batched(ReduceBatch b)
{
    const int64_t c = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    if (c >= b.first[b.n]) return;
    int j = 0;
    while (j + 1 < b.n && c >= b.first[j + 1]) j++;
    j = __builtin_amdgcn_readfirstlane(j);        // the same for the whole wave
    const int64_t col = c - b.first[j];
    const int l = threadIdx.x % kWave;
    const float *p = b.job[j].part + col * kMaxPartialRows;
    const int rows = b.job[j].rows;
    float s = 0.f;
    for (int r = l; r < rows; r += kWave) s += p[r];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_down(s, off, kWave);
    if (l == 0) {
        const int64_t nk = b.job[j].nk;
        if (col < nk) {
            const int64_t split = b.job[j].split;
            if (col < split) {
                if (col < b.job[j].valid0) b.job[j].gk[col] += s;
            }
            else if (col < 2 * split)
                b.job[j].gk_up[0][col - split] += s;
            else
                b.job[j].gk_up[1][col - 2 * split] += s;
        } else {
            b.job[j].gb[col - nk] += s;
        }
    }
}

}  // namespace

hipError_t reduce_columns_batch(const ReduceJob *jobs, int n, hipStream_t s)
{
    if (n <= 0) return hipSuccess;
    if (n > kReduceBatch) return hipErrorInvalidValue;
    ReduceBatch b;
    int64_t total = 0;
    for (int i = 0; i < n; i++) {
        if (jobs[i].rows < 0 || jobs[i].rows > kMaxPartialRows || jobs[i].ncols < jobs[i].nk || !jobs[i].part ||
            (jobs[i].nk > 0 && !jobs[i].gk) || (jobs[i].ncols > jobs[i].nk && !jobs[i].gb))
            return hipErrorInvalidValue;
        b.job[i] = jobs[i];
        b.first[i] = total;
        total += jobs[i].ncols;
    }
    for (int i = n; i < kReduceBatch; i++) b.job[i] = ReduceJob{nullptr, nullptr, nullptr, 0, 0, 0, {nullptr, nullptr}, 0, 0};
    for (int i = n; i <= kReduceBatch; i++) b.first[i] = total;
    b.n = n;
    if (total == 0) return hipSuccess;
    const int64_t blocks = (total + 256 / kWave - 1) / (256 / kWave);
    if (blocks > INT32_MAX) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(reduce_columns_batched, dim3((unsigned)blocks), dim3(256), 0, s, b);
    return hipGetLastError();
}

}  // namespace msd
