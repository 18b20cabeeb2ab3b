// Ahead-of-time instantiations of the matrix-core fused kernel matrix x
// coefficients kernel for all 16 (A loader, B loader) pairs.
#include <hip/hip_runtime.h>

#include "launch.hpp"
#include "gram_coefficients.hpp"

namespace kmc_host {

template <int LOAD_A, int LOAD_B>
static hipError_t launch_one(const kmc::KernelCoefficientsArgs &args, dim3 grid, hipStream_t stream)
{
    if (args.kernel.centre)
        return launch(kmc::gram_times_coefficients<LOAD_A, LOAD_B, true>, grid, dim3(kmc::BK_THREADS), stream, args);
    return launch(kmc::gram_times_coefficients<LOAD_A, LOAD_B>, grid, dim3(kmc::BK_THREADS), stream, args);
}

hipError_t launch_gram_coefficients(int load_a, int load_b, const kmc::KernelCoefficientsArgs &args, dim3 grid,
                                    hipStream_t stream)
{
    switch (load_a * 4 + load_b) {
    case 0: return launch_one<0, 0>(args, grid, stream);
    case 1: return launch_one<0, 1>(args, grid, stream);
    case 2: return launch_one<0, 2>(args, grid, stream);
    case 3: return launch_one<0, 3>(args, grid, stream);
    case 4: return launch_one<1, 0>(args, grid, stream);
    case 5: return launch_one<1, 1>(args, grid, stream);
    case 6: return launch_one<1, 2>(args, grid, stream);
    case 7: return launch_one<1, 3>(args, grid, stream);
    case 8: return launch_one<2, 0>(args, grid, stream);
    case 9: return launch_one<2, 1>(args, grid, stream);
    case 10: return launch_one<2, 2>(args, grid, stream);
    case 11: return launch_one<2, 3>(args, grid, stream);
    case 12: return launch_one<3, 0>(args, grid, stream);
    case 13: return launch_one<3, 1>(args, grid, stream);
    case 14: return launch_one<3, 2>(args, grid, stream);
    case 15: return launch_one<3, 3>(args, grid, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kmc_host
