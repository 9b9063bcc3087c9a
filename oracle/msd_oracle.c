/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle for the dilated conv (+ReLU) path:
 * a plain-C restatement of the reference's CUDA kernels, used by the tests,
 * the smoke check and the CPU-baseline leg of the benchmark as the thing the
 * GPU results are compared with.  It is never linked into, imported by or
 * called from the shipped library or package.
 *
 * What pins each function (tests/test_oracle.py):
 *   msd_oracle_reflect      numpy.pad(mode="symmetric") and a brute-force table
 *   conv_forward            torch conv on a symmetric-padded gather, constants,
 *                           interior vs stock dilated conv, golden fixtures
 *   conv_backward_x/k/bias  torch autograd through that composite, adjoint
 *                           identities, dense Jacobians on tiny images
 */
#include <stdint.h>
#include <stdlib.h>

/*
 * Symmetric index fold (edge voxel repeated): kernel_utils.cuh:30-38.
 * Valid for -n <= i < 2n, which the dilation <= size rule guarantees
 * (msd_custom_convolutions.cpp:39-52).
 */
int msd_oracle_reflect(int i, int n)
{
    if (i < 0)
        i = -i - 1;
    else if (i >= n)
        i = 2 * n - i - 1;
    return i;
}

#define T float
#define SFX f32
#include "msd_oracle_impl.h"
#undef T
#undef SFX

#define T double
#define SFX f64
#include "msd_oracle_impl.h"
#undef T
#undef SFX
