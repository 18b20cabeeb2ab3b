// One (inner operator, inner power) pair of the fused pairwise-reduction
// kernel, instantiated for all 16 (A loader, B loader) combinations.
// Compiled several times with different -DKMC_INNER_OP / -DKMC_INNER_POW.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "launch.hpp"
#include "build_kernel.hpp"
#include "build_kernel_scalar_b.hpp"
#include "../host/dispatch_rules.hpp"

#ifndef KMC_INNER_OP
#error "compile with -DKMC_INNER_OP=<0|1> -DKMC_INNER_POW=<0..4>"
#endif

#define KMC_CAT_(a, b, c, d) a##b##c##d
#define KMC_CAT(a, b, c, d) KMC_CAT_(a, b, c, d)
#define KMC_LAUNCHER_NAME KMC_CAT(launch_build_kernel_, KMC_INNER_OP, _, KMC_INNER_POW)

namespace kmc_host {

// Whether the call is one for build_kernel_scalar_b (its header says what the kernel assumes): enough tiles of
// 256 x 64 in every batch entry to fill the chip twice.  From a sweep against build_kernel / build_kernel_four_waves
// (their time / this kernel's, p = 1 and p = 2, K = 64 .. 4096): 2256 tiles (6000 x 6000) 1.02 .. 1.07 and 1.05 .. 1.10,
// 1876 (1000 x 30000) 1.01 .. 1.02 and 1.03 .. 1.07, 3776 (30000 x 2000) 1.04 .. 1.21, 55342 (30000 x 30000) 1.02 .. 1.05 and
// 1.05 .. 1.08; 1024 tiles (4096 x 4096) 0.96 .. 1.03, and batches of small entries lose: 8 x 2048 x 2048 0.95 .. 1.0,
// 64 x 512 x 512 0.91 .. 1.0 for p = 1.
// A panel against itself (the tiles of one triangle, each stored twice; ordinary kernel's time / this kernel's, p = 1 and
// p = 2, one box): 30000 x 1024, 27966 tiles, 1.02 and 1.05; 16384 x 512, 8320 tiles, 0.99 and 1.05; 8192 x 1024 0.90 and 1.02;
// 12000 x 128 1.03 and 1.05; 6000 x 512 level: taken from 16000 tiles on.
// KERMAC_AMD_SCALAR_B_MIN_TILES=n replaces the size rule by "at least n tiles over the batch, any k" (read on every
// call, so that a test can send small shapes to the kernel).
static bool scalar_b_applies(const kmc::BuildKernelArgs &args, int64_t *grid_width)
{
    if (args.k < 16 || args.k % kmc::BK_TILE_K != 0 || (args.n % kmc::SB_WAVE_N != 0 && !(args.panels & kmc::BK_PANELS_B_PADDED)) ||
        args.k_total != 0 || args.repair_only)
        return false;
    const int64_t tiles_m = (static_cast<int64_t>(args.m) + kmc::SB_TILE_M - 1) / kmc::SB_TILE_M;
    const int64_t tiles_n = (static_cast<int64_t>(args.n) + kmc::SB_TILE_N - 1) / kmc::SB_TILE_N;
    // a panel against itself: tile row r holds the tiles 0 .. 4 r + 3 that reach the diagonal or lie below it
    const int64_t tiles = args.symmetric ? 2 * (tiles_m - 1) * tiles_m + (4 * tiles_m < tiles_n ? 4 * tiles_m : tiles_n) : tiles_m * tiles_n;
    if (tiles > 0x7fffffff || (args.symmetric && args.m != args.n)) return false;
    *grid_width = tiles;
    if (args.panels & kmc::BK_PANELS_COPIED) return true;       // the host made the copies for this kernel
    const char *text = std::getenv("KERMAC_AMD_SCALAR_B_MIN_TILES");
    const int forced = text ? std::atoi(text) : 0;
    if (forced > 0) return tiles * args.l >= forced;
    return tiles >= (args.symmetric ? kmc_rules::DIRECT_SCALAR_B_MIN_TILES_SYMMETRIC : kmc_rules::DIRECT_SCALAR_B_MIN_TILES) &&
           args.k >= kmc_rules::DIRECT_SCALAR_B_MIN_K;
}

template <int LOAD_A, int LOAD_B>
static hipError_t launch_one(const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream)
{
    // absolute differences, their squares, cubes and fourth powers, of large problems whose rows are contiguous on both
    // sides: b in scalar registers
    if constexpr (LOAD_A == kmc::LOAD_COL_VEC && LOAD_B == kmc::LOAD_COL_VEC && KMC_INNER_OP == kmc::OP_DIFF &&
                  (KMC_INNER_POW == kmc::POW_ABS || KMC_INNER_POW == kmc::POW_SQUARE || KMC_INNER_POW == kmc::POW_ABS_CUBE ||
                   KMC_INNER_POW == kmc::POW_ABS_FOURTH)) {
        int64_t grid_width = 0;
        if (scalar_b_applies(args, &grid_width)) {
            kmc::BuildKernelArgs copy = args;
            copy.sample = nullptr;          // an ordinary launch computes everything
            const float *a = args.a, *b = args.b;
            float *c = args.c;
            void *kernel_args[] = {&copy, &a, &b, &c};
            return hipLaunchKernel(reinterpret_cast<const void *>(kmc::build_kernel_scalar_b<KMC_INNER_OP, KMC_INNER_POW>),
                                   dim3(static_cast<unsigned>(grid_width), args.l), dim3(kmc::BK_THREADS), kernel_args, 0, stream);
        }
    }
    // contiguous rows on both sides, a contraction long enough for the walk to set the time, and an inner term
    // without transcendentals (whose loop needs more registers): the variant compiled for four waves per SIMD
    if constexpr (LOAD_A == kmc::LOAD_COL_VEC && LOAD_B == kmc::LOAD_COL_VEC && KMC_INNER_POW != kmc::POW_POW) {
        if (args.k >= kmc_rules::DIRECT_FOUR_WAVES_MIN_K && !args.repair_only)
            return launch(kmc::build_kernel_four_waves<KMC_INNER_OP, KMC_INNER_POW>, grid, dim3(kmc::BK_THREADS), stream, args);
    }
    return launch(kmc::build_kernel<KMC_INNER_OP, KMC_INNER_POW, LOAD_A, LOAD_B>, grid, dim3(kmc::BK_THREADS), stream, args);
}

#if KMC_INNER_OP == 0 && KMC_INNER_POW == 2
// For a matrix-core call for squared differences that took a sample (args.sample): when the direct kernel with b in
// scalar registers can take the operands as they are, launches it in front of the repair launch, where it computes
// everything if the sample left the call to the direct kernel and exits at once if not.  Without it the repair launch
// does that work on the ordinary kernel, 8 % slower.  *launched says whether the call qualified.
hipError_t launch_scalar_b_if_the_sample_leaves(int load_a, int load_b, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *launched)
{
    *launched = false;
    int64_t grid_width = 0;
    if (!args.sample || load_a != kmc::LOAD_COL_VEC || load_b != kmc::LOAD_COL_VEC || !scalar_b_applies(args, &grid_width))
        return hipSuccess;
    kmc::BuildKernelArgs copy = args;
    const float *a = args.a, *b = args.b;
    float *c = args.c;
    void *kernel_args[] = {&copy, &a, &b, &c};
    *launched = true;
    return hipLaunchKernel(reinterpret_cast<const void *>(kmc::build_kernel_scalar_b<KMC_INNER_OP, KMC_INNER_POW>),
                           dim3(static_cast<unsigned>(grid_width), args.l), dim3(kmc::BK_THREADS), kernel_args, 0, stream);
}
#endif

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
