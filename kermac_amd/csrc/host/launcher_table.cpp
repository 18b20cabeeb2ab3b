// The ahead-of-time variant tables: which (inner operator, inner power) pairs
// are compiled into the library.  Must match AOT_BUILD_KERNEL_VARIANTS and
// AOT_COEFFICIENT_VARIANTS in kermac_amd/_build.py.  Other pairs are compiled at
// run time with hiprtc.
#include "launchers.hpp"

// Host-only data: skipped in the device compilation pass of this file.
#if !defined(__HIP_DEVICE_COMPILE__)
namespace kmc_host {

#define KMC_DECLARE_BUILD(op, pw) \
    hipError_t launch_build_kernel_##op##_##pw(int, int, const kmc::BuildKernelArgs &, dim3, hipStream_t);
#define KMC_DECLARE_COEF(op, pw) \
    hipError_t launch_kernel_coefficients_##op##_##pw(int, int, const kmc::KernelCoefficientsArgs &, dim3, hipStream_t);

KMC_DECLARE_BUILD(0, 0)  // DIFF, NOOP
KMC_DECLARE_BUILD(0, 1)  // DIFF, ABS      (L1 norm, Laplace-L1)
KMC_DECLARE_BUILD(0, 2)  // DIFF, SQUARE   (L2 norm, Laplace-L2, Gaussian)
KMC_DECLARE_BUILD(0, 4)  // DIFF, POW      (fractional p norm)
KMC_DECLARE_BUILD(0, 5)  // DIFF, |x|^0.5  (substituted for POW with a scalar exponent, see device_common.hpp)
KMC_DECLARE_BUILD(0, 6)  // DIFF, |x|^1.5
KMC_DECLARE_BUILD(0, 7)  // DIFF, |x|^3
KMC_DECLARE_BUILD(0, 8)  // DIFF, |x|^4
KMC_DECLARE_BUILD(1, 0)  // DOT,  NOOP     (plain a @ b.T)

KMC_DECLARE_COEF(0, 1)
KMC_DECLARE_COEF(0, 2)
KMC_DECLARE_COEF(0, 4)

const BuildLauncher build_launchers[] = {
    {0, 0, launch_build_kernel_0_0},
    {0, 1, launch_build_kernel_0_1},
    {0, 2, launch_build_kernel_0_2},
    {0, 4, launch_build_kernel_0_4},
    {0, 5, launch_build_kernel_0_5},
    {0, 6, launch_build_kernel_0_6},
    {0, 7, launch_build_kernel_0_7},
    {0, 8, launch_build_kernel_0_8},
    {1, 0, launch_build_kernel_1_0},
};
const int build_launcher_count = sizeof(build_launchers) / sizeof(build_launchers[0]);

const CoefLauncher coef_launchers[] = {
    {0, 1, launch_kernel_coefficients_0_1},
    {0, 2, launch_kernel_coefficients_0_2},
    {0, 4, launch_kernel_coefficients_0_4},
};
const int coef_launcher_count = sizeof(coef_launchers) / sizeof(coef_launchers[0]);

}  // namespace kmc_host
#endif
