// C-ABI entry point for the fused kernel-matrix x coefficients contraction.
#include "host_common.hpp"

using namespace kmc_host;

extern "C" int kmc_kernel_times_coefficients(const kmc_kernel_coefficients_params *params, void *stream)
{
    (void)params;
    (void)stream;
    return fail(KMC_ERR_UNSUPPORTED_VARIANT, "kmc_kernel_times_coefficients is not built yet");
}
