// Tables of the ahead-of-time compiled kernel instantiations.  Each entry is
// defined in its own device translation unit (kernels/*_inst.hip compiled once
// per (inner operator, inner power) pair).
#pragma once

#include <hip/hip_runtime.h>

#include "../kernels/kernel_coefficients.hpp"

namespace kmc_host {

typedef hipError_t (*build_launcher_fn)(int load_a, int load_b, const kmc::BuildKernelArgs &args, dim3 grid,
                                        hipStream_t stream);
typedef hipError_t (*coef_launcher_fn)(int load_a, int load_b, const kmc::KernelCoefficientsArgs &args, dim3 grid,
                                       hipStream_t stream);

struct BuildLauncher {
    int inner_operator;
    int inner_power;
    build_launcher_fn launch;
};

struct CoefLauncher {
    int inner_operator;
    int inner_power;
    coef_launcher_fn launch;
};

extern const BuildLauncher build_launchers[];
extern const int build_launcher_count;
extern const CoefLauncher coef_launchers[];
extern const int coef_launcher_count;

}  // namespace kmc_host
