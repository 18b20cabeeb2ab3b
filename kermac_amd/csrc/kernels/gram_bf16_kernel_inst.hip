// Ahead-of-time instantiations of the split-bf16 matrix-core L2 kernel for all 16
// (A loader, B loader) pairs, plus the ragged-K variants of the pairs with 128-bit row-major loads.
#include <hip/hip_runtime.h>

#include "launch.hpp"
#include "gram_bf16_kernel.hpp"

namespace kmc_host {

template <int LOAD_A, int LOAD_B>
static hipError_t launch_one(const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream)
{
    constexpr bool has_ragged_variant = LOAD_A == kmc::LOAD_ROW_VEC || LOAD_B == kmc::LOAD_ROW_VEC;
    hipError_t status;
    const bool ragged = has_ragged_variant && args.k % kmc::BK_TILE_K != 0;
    if (args.centre) {
        status = ragged ? launch(kmc::gram_bf16_l2_kernel<LOAD_A, LOAD_B, has_ragged_variant, true>, grid, dim3(kmc::BK_THREADS), stream, args)
                        : launch(kmc::gram_bf16_l2_kernel<LOAD_A, LOAD_B, false, true>, grid, dim3(kmc::BK_THREADS), stream, args);
    } else {
        status = ragged ? launch(kmc::gram_bf16_l2_kernel<LOAD_A, LOAD_B, has_ragged_variant>, grid, dim3(kmc::BK_THREADS), stream, args)
                        : launch(kmc::gram_bf16_l2_kernel<LOAD_A, LOAD_B>, grid, dim3(kmc::BK_THREADS), stream, args);
    }
    return status;
}

hipError_t launch_gram_bf16_l2(int load_a, int load_b, const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream)
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
