// Ahead-of-time instantiations of the kernel-gradient contraction: 3 norm types
// x (vector-ALU kernel with 1 to 6 or 8 outputs per lane tile, matrix-core kernel with
// 16 or 32 output columns, with and without a partial last K slice).
#include <hip/hip_runtime.h>

#include "launch.hpp"
#include "norm_gradient_mfma.hpp"

namespace kmc_host {

template <int NORM>
static hipError_t launch_norm(int o_tile, const kmc::NormGradientArgs &args, dim3 grid, hipStream_t stream)
{
    const dim3 block(kmc::NG_THREADS);
    const bool k_tail = args.k % kmc::NGM_TILE_K != 0;
    hipError_t status;
    switch (o_tile) {
    case 1: status = launch(kmc::norm_kernel_gradient<NORM, 1>, grid, block, stream, args); break;
    case 2: status = launch(kmc::norm_kernel_gradient<NORM, 2>, grid, block, stream, args); break;
    case 3: status = launch(kmc::norm_kernel_gradient<NORM, 3>, grid, block, stream, args); break;
    case 4: status = launch(kmc::norm_kernel_gradient<NORM, 4>, grid, block, stream, args); break;
    case 5: status = launch(kmc::norm_kernel_gradient<NORM, 5>, grid, block, stream, args); break;
    case 6: status = launch(kmc::norm_kernel_gradient<NORM, 6>, grid, block, stream, args); break;
    case 8: status = launch(kmc::norm_kernel_gradient<NORM, 8>, grid, block, stream, args); break;
    case 16:
        if (k_tail) status = launch(kmc::norm_kernel_gradient_mfma<NORM, 1, true>, grid, block, stream, args);
        else status = launch(kmc::norm_kernel_gradient_mfma<NORM, 1, false>, grid, block, stream, args);
        break;
    case 32:
        if (k_tail) status = launch(kmc::norm_kernel_gradient_mfma<NORM, 2, true>, grid, block, stream, args);
        else status = launch(kmc::norm_kernel_gradient_mfma<NORM, 2, false>, grid, block, stream, args);
        break;
    default: return hipErrorInvalidValue;
    }
    return status;
}

hipError_t launch_norm_gradient(int norm_type, int o_tile, const kmc::NormGradientArgs &args, dim3 grid,
                                hipStream_t stream)
{
    switch (norm_type) {
    case kmc::NORM_L1: return launch_norm<kmc::NORM_L1>(o_tile, args, grid, stream);
    case kmc::NORM_L2: return launch_norm<kmc::NORM_L2>(o_tile, args, grid, stream);
    case kmc::NORM_P: return launch_norm<kmc::NORM_P>(o_tile, args, grid, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kmc_host
