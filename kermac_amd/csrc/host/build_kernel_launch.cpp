// C-ABI entry points for the fused pairwise-reduction kernel: argument checks,
// loader selection, and dispatch to the ahead-of-time instantiations (or to a
// run-time compiled function).
#include "host_common.hpp"
#include "../kernels/build_kernel.hpp"
#include "launchers.hpp"

#include <climits>

using namespace kmc_host;

namespace {

int check_operand(const char *name, const float *ptr, int rows, int k, int64_t ld, int64_t bs, int majorness, int l)
{
    if (majorness != KMC_COL_MAJOR && majorness != KMC_ROW_MAJOR)
        return fail(KMC_ERR_INVALID_ARGUMENT, "%s: majorness %d is not a kmc_majorness", name, majorness);
    if (rows > 0 && k > 0 && !ptr) return fail(KMC_ERR_INVALID_ARGUMENT, "%s: null pointer", name);
    const int contiguous_extent = majorness == KMC_COL_MAJOR ? rows : k;
    const int strided_extent = majorness == KMC_COL_MAJOR ? k : rows;
    if (strided_extent > 1 && ld < contiguous_extent)
        return fail(KMC_ERR_INVALID_ARGUMENT, "%s: leading dimension %lld is smaller than the contiguous extent %d",
                    name, static_cast<long long>(ld), contiguous_extent);
    if (ld < 0 || bs < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "%s: negative stride", name);
    (void)l;
    return KMC_OK;
}

int pick_load_mode(const float *ptr, int64_t ld, int64_t bs, int majorness, int flags)
{
    const bool vec = !(flags & KMC_FLAG_FORCE_SCALAR_ACCESS) && aligned16(ptr) && ld % 4 == 0 && bs % 4 == 0;
    if (majorness == KMC_COL_MAJOR) return vec ? kmc::LOAD_COL_VEC : kmc::LOAD_COL_SCALAR;
    return vec ? kmc::LOAD_ROW_VEC : kmc::LOAD_ROW_SCALAR;
}

// Validates `p` and fills the device argument block.  `need_c` is false for the
// fused coefficient kernel, which never stores the m x n matrix.
int prepare(const kmc_build_kernel_params *p, bool need_c, kmc::BuildKernelArgs *args, int *load_a, int *load_b)
{
    if (!p) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    if (p->inner_operator != KMC_OP_DIFF && p->inner_operator != KMC_OP_DOT)
        return fail(KMC_ERR_INVALID_ARGUMENT, "inner_operator %d is not a kmc_inner_operator", p->inner_operator);
    if (p->inner_power < KMC_POW_NOOP || p->inner_power > KMC_POW_POW)
        return fail(KMC_ERR_INVALID_ARGUMENT, "inner_power %d is not a kmc_power_type", p->inner_power);
    if (p->outer_power < KMC_POW_NOOP || p->outer_power > KMC_POW_POW)
        return fail(KMC_ERR_INVALID_ARGUMENT, "outer_power %d is not a kmc_power_type", p->outer_power);
    if (p->kernel_type < KMC_KERNEL_NONE || p->kernel_type > KMC_KERNEL_GAUSSIAN)
        return fail(KMC_ERR_INVALID_ARGUMENT, "kernel_type %d is not a kmc_kernel_type", p->kernel_type);
    if (p->m < 0 || p->n < 0 || p->k < 0 || p->l < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative extent (m=%d n=%d k=%d l=%d)", p->m, p->n, p->k, p->l);
    if (p->l > 65535) return fail(KMC_ERR_INVALID_ARGUMENT, "batch count %d exceeds 65535", p->l);
    int status = check_operand("a", p->a, p->m, p->k, p->a_ld, p->a_bs, p->a_majorness, p->l);
    if (status != KMC_OK) return status;
    status = check_operand("b", p->b, p->n, p->k, p->b_ld, p->b_bs, p->b_majorness, p->l);
    if (status != KMC_OK) return status;
    if (need_c) {
        if (p->m > 0 && p->n > 0 && !p->c) return fail(KMC_ERR_INVALID_ARGUMENT, "c: null pointer");
        if (p->n > 1 && p->c_ld < p->m)
            return fail(KMC_ERR_INVALID_ARGUMENT, "c: leading dimension %lld is smaller than m=%d",
                        static_cast<long long>(p->c_ld), p->m);
        if (p->c_ld < 0 || p->c_bs < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "c: negative stride");
    }
    const int64_t tiles_m = ceil_div(p->m, kmc::BK_TILE_M);
    const int64_t tiles_n = ceil_div(p->n, kmc::BK_TILE_N);
    // Rounding the n tiles up to a multiple of 8 keeps every n tile on one XCD (see
    // tile_of_workgroup).  The padding workgroups exit at once but still take their turn
    // in the dispatch order, so the rounding is dropped where it would add more than one
    // workgroup in eight: those problems are small enough for every L2 to hold the panels.
    // (Measured: 16 tiles padded to 32 per batch entry, as a batch of 32, left half the CUs
    // idle: 0.255 ms against 0.167 ms without the padding; 1000 problems of one tile each,
    // padded to 8: 0.283 against 0.099 ms.)
    int64_t tiles_n_padded = (tiles_n + kmc::BK_XCDS - 1) / kmc::BK_XCDS * kmc::BK_XCDS;
    if ((tiles_n_padded - tiles_n) * 8 > tiles_n) tiles_n_padded = tiles_n;
    if (tiles_m * tiles_n_padded > INT_MAX) return fail(KMC_ERR_INVALID_ARGUMENT, "m x n needs more than 2^31 tiles");

    args->m = p->m; args->n = p->n; args->k = p->k; args->l = p->l;
    args->a = p->a; args->a_ld = p->a_ld; args->a_bs = p->a_bs;
    args->b = p->b; args->b_ld = p->b_ld; args->b_bs = p->b_bs;
    args->c = p->c; args->c_ld = p->c_ld; args->c_bs = p->c_bs;
    args->p_inner = p->p_inner; args->p_inner_bs = p->p_inner_bs; args->p_inner_value = p->p_inner_value;
    args->p_outer = p->p_outer; args->p_outer_bs = p->p_outer_bs; args->p_outer_value = p->p_outer_value;
    args->bandwidth = p->bandwidth; args->bandwidth_bs = p->bandwidth_bs; args->bandwidth_value = p->bandwidth_value;
    args->regularization = p->regularization; args->regularization_bs = p->regularization_bs;
    args->regularization_value = p->regularization_value;
    args->reg_off_x = p->regularization_offset_x;
    args->reg_off_y = p->regularization_offset_y;
    args->epsilon = p->epsilon;
    args->diff_sign = (p->flags & KMC_FLAG_NEGATE_DIFF) ? -1.0f : 1.0f;
    args->repair_only = 0;
    // Same panel on both sides, same offsets, and an inner term that does not change
    // when its operands are exchanged (every DOT term; |x|, x^2, |x|^p of a
    // difference): C(n, m) equals C(m, n) bit for bit, so half the tiles suffice.
    const bool exchangeable = p->inner_operator == KMC_OP_DOT || p->inner_power == KMC_POW_ABS ||
                              p->inner_power == KMC_POW_SQUARE || p->inner_power == KMC_POW_POW;
    args->symmetric = need_c && !(p->flags & KMC_FLAG_NO_SYMMETRY) && exchangeable && p->a == p->b && p->m == p->n &&
                      p->a_ld == p->b_ld && p->a_bs == p->b_bs && p->a_majorness == p->b_majorness &&
                      p->regularization_offset_x == p->regularization_offset_y && tiles_m > 1;
    args->gram_trust = p->gram_trust > 0.0f ? p->gram_trust : 0.25f;
    if (p->k_total < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "negative k_total %d", p->k_total);
    if (p->k_total > 0) {
        // the batch entries are ranges of one contraction: all but the last are full
        const int64_t before_last = static_cast<int64_t>(p->l - 1) * p->k;
        if (p->l < 1 || p->k < 1 || before_last >= p->k_total || before_last + p->k < p->k_total)
            return fail(KMC_ERR_INVALID_ARGUMENT, "k_total=%d is not covered by l=%d ranges of k=%d, the last one not empty",
                        p->k_total, p->l, p->k);
        if (p->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16 | KMC_FLAG_DOT_PIECES))
            return fail(KMC_ERR_INVALID_ARGUMENT, "k_total cannot be combined with the matrix-core flags");
    }
    args->k_total = p->k_total;
    args->centre = nullptr;
    args->centre_bs = 0;
    args->sample = nullptr;
    args->panels = 0;
    if ((p->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16)) && p->gram_centre) {
        if (!aligned16(p->gram_centre) || p->gram_centre_bs % 4 != 0 || p->gram_centre_bs < 0)
            return fail(KMC_ERR_INVALID_ARGUMENT, "gram_centre must be 16-byte aligned with a batch stride that is a multiple of 4");
        args->centre = p->gram_centre;
        args->centre_bs = p->gram_centre_bs;
    }
    args->outer_power = p->outer_power;
    args->kernel_type = p->kernel_type;
    args->c_vec = need_c && !(p->flags & KMC_FLAG_FORCE_SCALAR_ACCESS) && aligned16(p->c) && p->c_ld % 4 == 0 &&
                  p->c_bs % 4 == 0;
    args->tiles_m = static_cast<int>(tiles_m);
    args->tiles_n = static_cast<int>(tiles_n);
    args->tiles_n_padded = static_cast<int>(tiles_n_padded);
    args->grid_width = static_cast<int>(args->symmetric ? tiles_m * (tiles_m + 1) / 2 : tiles_m * tiles_n_padded);
    *load_a = pick_load_mode(p->a, p->a_ld, p->a_bs, p->a_majorness, p->flags);
    *load_b = pick_load_mode(p->b, p->b_ld, p->b_bs, p->b_majorness, p->flags);
    return KMC_OK;
}

kmc_host::build_launcher_fn find_launcher(int inner_operator, int inner_power)
{
    for (int i = 0; i < kmc_host::build_launcher_count; i++) {
        const kmc_host::BuildLauncher &entry = kmc_host::build_launchers[i];
        if (entry.inner_operator == inner_operator && entry.inner_power == inner_power) return entry.launch;
    }
    return nullptr;
}

}  // namespace

namespace kmc_host {
hipError_t launch_gram_l2(int load_a, int load_b, const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream);
hipError_t launch_gram_bf16_l2(int load_a, int load_b, const kmc::BuildKernelArgs &args, dim3 grid, hipStream_t stream);
int64_t gram_f16_wide_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args);
hipError_t launch_gram_f16_wide(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *taken,
                                const unsigned **sample = nullptr);
hipError_t launch_scalar_b_if_the_sample_leaves(int load_a, int load_b, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *launched);
hipError_t launch_gram_probe(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, unsigned *sample, hipStream_t stream);
int64_t l1_fixed_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args);
hipError_t launch_l1_fixed(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *taken);
int64_t direct_panels_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args);
hipError_t launch_direct_panels(const kmc_build_kernel_params *p, kmc::BuildKernelArgs *args, hipStream_t stream, bool *taken);
hipError_t launch_finish_partials(const kmc::BuildKernelArgs &kernel, const float *partials, int64_t partial_ld,
                                  int64_t partial_bs, int64_t partial_slice, int slices, int vec, hipStream_t stream);
}

namespace kmc_host {
int prepare_build_kernel(const kmc_build_kernel_params *p, bool need_c, kmc::BuildKernelArgs *args, int *load_a, int *load_b)
{
    return prepare(p, need_c, args, load_a, load_b);
}
}  // namespace kmc_host

extern "C" {

int kmc_build_kernel_has_variant(int32_t inner_operator, int32_t inner_power)
{
    // the special exponents (device_common.hpp, SpecialPower) are internal, not variants a caller can ask for
    return inner_power <= KMC_POW_POW && find_launcher(inner_operator, inner_power) != nullptr;
}

int kmc_build_kernel_load_modes(const kmc_build_kernel_params *params, int32_t *load_a, int32_t *load_b)
{
    kmc::BuildKernelArgs args;
    int la = 0, lb = 0;
    int status = prepare(params, false, &args, &la, &lb);   // only a and b matter here
    if (status != KMC_OK) return status;
    if (load_a) *load_a = la;
    if (load_b) *load_b = lb;
    return KMC_OK;
}

int kmc_gram_workspace_bytes(const kmc_build_kernel_params *params, int64_t *bytes)
{
    if (!bytes) return fail(KMC_ERR_INVALID_ARGUMENT, "bytes: null pointer");
    if (!params) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    // the result may not be allocated yet when the caller asks: any address stands in for it
    kmc_build_kernel_params asked = *params;
    if (!asked.c) asked.c = reinterpret_cast<float *>(static_cast<uintptr_t>(256));
    kmc::BuildKernelArgs args;
    int load_a = 0, load_b = 0;
    int status = prepare(&asked, true, &args, &load_a, &load_b);
    if (status != KMC_OK) return status;
    *bytes = gram_f16_wide_bytes(&asked, args);
    if (*bytes == 0) *bytes = l1_fixed_bytes(&asked, args);
    if (*bytes == 0) *bytes = direct_panels_bytes(&asked, args);
    return KMC_OK;
}

int kmc_build_kernel(const kmc_build_kernel_params *params, void *stream)
{
    kmc::BuildKernelArgs args;
    int load_a = 0, load_b = 0;
    int status = prepare(params, true, &args, &load_a, &load_b);
    if (status != KMC_OK) return status;
    int inner_power = params->inner_power;
    if (params->inner_operator == KMC_OP_DIFF && inner_power == KMC_POW_POW && !params->p_inner &&
        !(params->flags & KMC_FLAG_GENERIC_POWER)) {
        // Scalar exponents with a cheaper exact form (device_common.hpp, SpecialPower).
        const float p = params->p_inner_value;
        const int special = p == 0.5f ? kmc::POW_ABS_HALF : p == 1.5f ? kmc::POW_ABS_THREE_HALVES
                          : p == 3.0f ? kmc::POW_ABS_CUBE : p == 4.0f ? kmc::POW_ABS_FOURTH : inner_power;
        if (find_launcher(params->inner_operator, special)) inner_power = special;
    }
    kmc_host::build_launcher_fn launch = find_launcher(params->inner_operator, inner_power);
    if (!launch) {
        return fail(KMC_ERR_UNSUPPORTED_VARIANT,
                    "inner_operator=%d inner_power=%d is not compiled ahead of time; compile it at run time",
                    params->inner_operator, params->inner_power);
    }
    if (args.m == 0 || args.n == 0 || args.l == 0) return KMC_OK;
    status = require_gfx950();
    if (status != KMC_OK) return status;
    const dim3 grid(static_cast<unsigned>(args.grid_width), args.l, 1);
    if (params->flags & KMC_FLAG_DOT_PIECES) {
        if (params->inner_operator != KMC_OP_DOT || params->inner_power != KMC_POW_NOOP)
            return fail(KMC_ERR_INVALID_ARGUMENT, "KMC_FLAG_DOT_PIECES needs inner_operator DOT and inner_power NOOP");
        if (params->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16))
            return fail(KMC_ERR_INVALID_ARGUMENT, "KMC_FLAG_DOT_PIECES cannot be combined with KMC_FLAG_L2_GRAM");
        bool wide = false;
        hipError_t g = launch_gram_f16_wide(params, args, static_cast<hipStream_t>(stream), &wide);
        if (g != hipSuccess) return fail_hip(g, "gram_f16_wide launches");
        if (wide) return KMC_OK;
    }
    if (params->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16)) {
        if (params->inner_operator != KMC_OP_DIFF || params->inner_power != KMC_POW_SQUARE)
            return fail(KMC_ERR_INVALID_ARGUMENT, "KMC_FLAG_L2_GRAM needs inner_operator DIFF and inner_power SQUARE");
        // Matrix-core pass over every tile, then the direct kernel over the tiles it marked.
        bool wide = false;
        const unsigned *sample_taken = nullptr;
        hipError_t g = launch_gram_f16_wide(params, args, static_cast<hipStream_t>(stream), &wide, &sample_taken);
        if (g != hipSuccess) return fail_hip(g, "gram_f16_wide launches");
        if (wide) args.sample = sample_taken;
        if (!wide) {
            // The one-step kernels: with KMC_SAMPLE_BYTES of workspace, a sample of the result first (gram_probe.hip),
            // so that data whose near-duplicates sit in every tile costs the direct kernel's time, not both.
            if (!(params->flags & KMC_FLAG_NO_PROBE) && params->gram_workspace && params->gram_workspace_bytes >= KMC_SAMPLE_BYTES &&
                (reinterpret_cast<uintptr_t>(params->gram_workspace) & 255) == 0 && args.k > 0) {
                unsigned *sample = static_cast<unsigned *>(params->gram_workspace);
                g = launch_gram_probe(params, args, sample, static_cast<hipStream_t>(stream));
                if (g != hipSuccess) return fail_hip(g, "gram_probe_operands launch");
                args.sample = sample;
            }
            g = (params->flags & KMC_FLAG_L2_GRAM_BF16)
                    ? launch_gram_bf16_l2(load_a, load_b, args, grid, static_cast<hipStream_t>(stream))
                    : launch_gram_l2(load_a, load_b, args, grid, static_cast<hipStream_t>(stream));
            if (g != hipSuccess) return fail_hip(g, "gram_l2_kernel launch");
        }
        if (args.sample) {
            // Where the sample left the call to the direct kernel, its fastest variant does the work (if it can take
            // these operands), and the repair launch behind it finds nothing to do.
            bool launched = false;
            g = launch_scalar_b_if_the_sample_leaves(load_a, load_b, args, static_cast<hipStream_t>(stream), &launched);
            if (g != hipSuccess) return fail_hip(g, "build_kernel_scalar_b launch");
            args.sample = nullptr;
        }
        args.repair_only = 1;
    }
    if (params->flags & KMC_FLAG_L1_FIXED) {
        if (params->inner_operator != KMC_OP_DIFF || params->inner_power != KMC_POW_ABS)
            return fail(KMC_ERR_INVALID_ARGUMENT, "KMC_FLAG_L1_FIXED needs inner_operator DIFF and inner_power ABS");
        // Fixed-point pass over every tile, then the direct kernel over the tiles it marked.
        bool fixed = false;
        hipError_t g = launch_l1_fixed(params, args, static_cast<hipStream_t>(stream), &fixed);
        if (g != hipSuccess) return fail_hip(g, "l1_fixed launches");
        if (fixed) args.repair_only = 1;
    }
    if (params->flags & KMC_FLAG_DIRECT_PANELS) {
        // Large absolute- and squared-difference problems whose operands the kernel with b in scalar registers cannot
        // take as they are: copies that it can (panel_copy.hip), then the ordinary launch on the copies.
        bool copied = false;
        hipError_t g = launch_direct_panels(params, &args, static_cast<hipStream_t>(stream), &copied);
        if (g != hipSuccess) return fail_hip(g, "panel_copy launches");
        if (copied) load_a = load_b = kmc::LOAD_COL_VEC;
    }
    hipError_t e = launch(load_a, load_b, args, grid, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(e, "build_kernel launch");
    return KMC_OK;
}

int kmc_build_kernel_finish(const kmc_build_kernel_params *params, const float *partials, int64_t partial_ld,
                            int64_t partial_bs, int64_t partial_slice, int32_t slices, void *stream)
{
    kmc::BuildKernelArgs args;
    int load_a = 0, load_b = 0;
    int status = prepare(params, true, &args, &load_a, &load_b);
    if (status != KMC_OK) return status;
    if (slices < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "negative slice count %d", slices);
    if (args.m == 0 || args.n == 0 || args.l == 0) return KMC_OK;
    if (slices > 0 && !partials) return fail(KMC_ERR_INVALID_ARGUMENT, "partials: null pointer");
    if (partial_ld < args.m && args.n > 1)
        return fail(KMC_ERR_INVALID_ARGUMENT, "partials: leading dimension %lld is smaller than m=%d",
                    static_cast<long long>(partial_ld), args.m);
    if (partial_ld < 0 || partial_bs < 0 || partial_slice < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "partials: negative stride");
    status = require_gfx950();
    if (status != KMC_OK) return status;
    const int vec = args.c_vec && aligned16(partials) && partial_ld % 4 == 0 && partial_bs % 4 == 0 && partial_slice % 4 == 0;
    hipError_t e = launch_finish_partials(args, partials, partial_ld, partial_bs, partial_slice, slices, vec,
                                          static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(e, "finish_partials launch");
    return KMC_OK;
}

int kmc_build_kernel_jit(void *function, const kmc_build_kernel_params *params, void *stream)
{
    if (!function) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_build_kernel_jit: null function");
    kmc::BuildKernelArgs args;
    int load_a = 0, load_b = 0;
    int status = prepare(params, true, &args, &load_a, &load_b);
    if (status != KMC_OK) return status;
    if (args.m == 0 || args.n == 0 || args.l == 0) return KMC_OK;
    status = require_gfx950();
    if (status != KMC_OK) return status;
    size_t size = sizeof(args);
    void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    hipError_t e = hipModuleLaunchKernel(static_cast<hipFunction_t>(function),
                                         static_cast<unsigned>(args.grid_width),
                                         args.l, 1, kmc::BK_THREADS, 1, 1, 0, static_cast<hipStream_t>(stream), nullptr,
                                         config);
    if (e != hipSuccess) return fail_hip(e, "build_kernel (run-time compiled) launch");
    return KMC_OK;
}

}  // extern "C"
