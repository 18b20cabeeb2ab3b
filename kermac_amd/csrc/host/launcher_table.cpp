// The ahead-of-time variant table: which (inner operator, inner power) pairs
// are compiled into the library.  Must match AOT_BUILD_KERNEL_VARIANTS in
// kermac_amd/_build.py.  Other pairs are compiled at run time with hiprtc.
#include "launchers.hpp"

// Host-only data: skipped in the device compilation pass of this file.
#if !defined(__HIP_DEVICE_COMPILE__)
namespace kmc_host {

#define KMC_DECLARE(op, pw) \
    hipError_t launch_build_kernel_##op##_##pw(int, int, const kmc::BuildKernelArgs &, dim3, hipStream_t);

KMC_DECLARE(0, 0)  // DIFF, NOOP
KMC_DECLARE(0, 1)  // DIFF, ABS      (L1 norm, Laplace-L1)
KMC_DECLARE(0, 2)  // DIFF, SQUARE   (L2 norm, Laplace-L2, Gaussian)
KMC_DECLARE(0, 4)  // DIFF, POW      (fractional p norm)
KMC_DECLARE(1, 0)  // DOT,  NOOP     (plain a @ b.T)

const BuildLauncher build_launchers[] = {
    {0, 0, launch_build_kernel_0_0},
    {0, 1, launch_build_kernel_0_1},
    {0, 2, launch_build_kernel_0_2},
    {0, 4, launch_build_kernel_0_4},
    {1, 0, launch_build_kernel_1_0},
};
const int build_launcher_count = sizeof(build_launchers) / sizeof(build_launchers[0]);

}  // namespace kmc_host
#endif
