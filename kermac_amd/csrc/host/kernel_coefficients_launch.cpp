// C-ABI entry points for the fused kernel-matrix x coefficients contraction.
#include "host_common.hpp"
#include "../kernels/kernel_coefficients.hpp"
#include "launchers.hpp"

using namespace kmc_host;

namespace kmc_host {
int prepare_build_kernel(const kmc_build_kernel_params *p, bool need_c, kmc::BuildKernelArgs *args, int *load_a,
                         int *load_b);
hipError_t launch_gram_coefficients(int load_a, int load_b, const kmc::KernelCoefficientsArgs &args, dim3 grid,
                                    hipStream_t stream);
}

namespace {

// `wide_allowed`: the launch goes to an ahead-of-time instantiation of the vector kernel,
// which exists for 32 and for 64 coefficient columns per workgroup; the matrix-core
// variant and run-time compiled functions hold 32.
int prepare(const kmc_kernel_coefficients_params *p, bool wide_allowed, kmc::KernelCoefficientsArgs *kc, int *load_a,
            int *load_b, dim3 *grid, bool *empty)
{
    if (!p) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    int status = prepare_build_kernel(&p->kernel, false, &kc->kernel, load_a, load_b);
    if (status != KMC_OK) return status;
    if (p->o < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "negative coefficient column count %d", p->o);
    if (p->kernel.k_total != 0) return fail(KMC_ERR_INVALID_ARGUMENT, "k_total is for kmc_build_kernel only");
    const kmc::BuildKernelArgs &k = kc->kernel;
    *empty = k.m == 0 || k.l == 0 || p->o == 0;
    if (*empty) return KMC_OK;
    if (!p->out || (k.n > 0 && !p->coef)) return fail(KMC_ERR_INVALID_ARGUMENT, "null coef / out pointer");
    if ((k.n > 1 && p->coef_ld < p->o) || (k.m > 1 && p->out_ld < p->o))
        return fail(KMC_ERR_INVALID_ARGUMENT, "coef / out leading dimension is smaller than o=%d", p->o);
    if (p->coef_ld < 0 || p->coef_bs < 0 || p->out_ld < 0 || p->out_bs < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative stride");
    kc->o = p->o;
    kc->columns = wide_allowed && p->o > kmc::KC_COLUMNS ? 64 : kmc::KC_COLUMNS;
    kc->o_chunks = ceil_div(p->o, kc->columns);
    kc->coef = p->coef; kc->coef_ld = p->coef_ld; kc->coef_bs = p->coef_bs;
    kc->out = p->out; kc->out_ld = p->out_ld; kc->out_bs = p->out_bs;
    kc->coef_vec = !(p->kernel.flags & KMC_FLAG_FORCE_SCALAR_ACCESS) && aligned16(p->coef) && p->coef_ld % 4 == 0 &&
                   p->coef_bs % 4 == 0;
    const int64_t grid_y = static_cast<int64_t>(k.l) * kc->o_chunks;
    if (grid_y > 65535)
        return fail(KMC_ERR_INVALID_ARGUMENT, "batch x coefficient chunks = %lld exceeds 65535", static_cast<long long>(grid_y));
    if (p->n_ranges < 0 || p->n_ranges > 65535)
        return fail(KMC_ERR_INVALID_ARGUMENT, "n_ranges = %d is outside 0 .. 65535", p->n_ranges);
    const int ranges = p->n_ranges > 1 ? p->n_ranges : 1;
    if (ranges > 1 && p->out_range_stride < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "negative out_range_stride");
    kc->split_tiles = k.tiles_n > 0 ? ceil_div(k.tiles_n, ranges) : 1;
    kc->out_split_stride = ranges > 1 ? p->out_range_stride : 0;
    *grid = dim3(k.tiles_m, static_cast<unsigned>(grid_y), static_cast<unsigned>(ranges));
    return KMC_OK;
}

kmc_host::coef_launcher_fn find_launcher(int inner_operator, int inner_power)
{
    for (int i = 0; i < kmc_host::coef_launcher_count; i++) {
        const kmc_host::CoefLauncher &entry = kmc_host::coef_launchers[i];
        if (entry.inner_operator == inner_operator && entry.inner_power == inner_power) return entry.launch;
    }
    return nullptr;
}

}  // namespace

extern "C" {

int kmc_kernel_times_coefficients_has_variant(int32_t inner_operator, int32_t inner_power)
{
    return find_launcher(inner_operator, inner_power) != nullptr;
}

int kmc_kernel_times_coefficients(const kmc_kernel_coefficients_params *params, void *stream)
{
    kmc::KernelCoefficientsArgs kc;
    int load_a = 0, load_b = 0;
    dim3 grid;
    bool empty = false;
    const bool matrix_core = params && (params->kernel.flags & KMC_FLAG_L2_GRAM);
    int status = prepare(params, !matrix_core, &kc, &load_a, &load_b, &grid, &empty);
    if (status != KMC_OK) return status;
    kmc_host::coef_launcher_fn launch = find_launcher(params->kernel.inner_operator, params->kernel.inner_power);
    if (params->kernel.flags & KMC_FLAG_L2_GRAM) {
        if (params->kernel.inner_operator != KMC_OP_DIFF || params->kernel.inner_power != KMC_POW_SQUARE)
            return fail(KMC_ERR_INVALID_ARGUMENT, "KMC_FLAG_L2_GRAM needs inner_operator DIFF and inner_power SQUARE");
        launch = kmc_host::launch_gram_coefficients;   // kernel values from the matrix cores
    }
    if (!launch) {
        return fail(KMC_ERR_UNSUPPORTED_VARIANT,
                    "inner_operator=%d inner_power=%d is not compiled ahead of time; compile it at run time",
                    params->kernel.inner_operator, params->kernel.inner_power);
    }
    if (empty) return KMC_OK;
    status = require_gfx950();
    if (status != KMC_OK) return status;
    hipError_t e = launch(load_a, load_b, kc, grid, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(e, "kernel_times_coefficients launch");
    return KMC_OK;
}

int kmc_kernel_times_coefficients_jit(void *function, const kmc_kernel_coefficients_params *params, void *stream)
{
    if (!function) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_kernel_times_coefficients_jit: null function");
    kmc::KernelCoefficientsArgs kc;
    int load_a = 0, load_b = 0;
    dim3 grid;
    bool empty = false;
    int status = prepare(params, false, &kc, &load_a, &load_b, &grid, &empty);
    if (status != KMC_OK) return status;
    if (empty) return KMC_OK;
    status = require_gfx950();
    if (status != KMC_OK) return status;
    size_t size = sizeof(kc);
    void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &kc, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    hipError_t e = hipModuleLaunchKernel(static_cast<hipFunction_t>(function), grid.x, grid.y, grid.z, kmc::BK_THREADS, 1, 1,
                                         0, static_cast<hipStream_t>(stream), nullptr, config);
    if (e != hipSuccess) return fail_hip(e, "kernel_times_coefficients (run-time compiled) launch");
    return KMC_OK;
}

}  // extern "C"
