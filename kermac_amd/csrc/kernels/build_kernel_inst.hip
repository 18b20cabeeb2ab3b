// One (inner operator, inner power) pair of the fused pairwise-reduction
// kernel, instantiated for all 16 (A loader, B loader) combinations.
// Compiled several times with different -DKMC_INNER_OP / -DKMC_INNER_POW.
#include <hip/hip_runtime.h>

#include "launch.hpp"
#include "build_kernel.hpp"
#include "../host/dispatch_rules.hpp"

#ifndef KMC_INNER_OP
#error "compile with -DKMC_INNER_OP=<0|1> -DKMC_INNER_POW=<0..4>"
#endif

#define KMC_CAT_(a, b, c, d) a##b##c##d
#define KMC_CAT(a, b, c, d) KMC_CAT_(a, b, c, d)
#define KMC_LAUNCHER_NAME KMC_CAT(launch_build_kernel_, KMC_INNER_OP, _, KMC_INNER_POW)

namespace kmc_host {

template <int LOAD_A, int LOAD_B>
static hipError_t launch_one(const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream)
{
    // contiguous rows on both sides, a contraction long enough for the walk to set the time, and an inner term
    // without transcendentals (whose loop needs more registers): the variant compiled for four waves per SIMD
    if constexpr (LOAD_A == kmc::LOAD_COL_VEC && LOAD_B == kmc::LOAD_COL_VEC && KMC_INNER_POW != kmc::POW_POW) {
        if (args.k >= kmc_rules::DIRECT_FOUR_WAVES_MIN_K && !args.repair_only)
            return launch(kmc::build_kernel_four_waves<KMC_INNER_OP, KMC_INNER_POW>, grid, dim3(kmc::BK_THREADS), stream, args);
    }
    return launch(kmc::build_kernel<KMC_INNER_OP, KMC_INNER_POW, LOAD_A, LOAD_B>, grid, dim3(kmc::BK_THREADS), stream, args);
}

hipError_t KMC_LAUNCHER_NAME(int load_a, int load_b, const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream)
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
