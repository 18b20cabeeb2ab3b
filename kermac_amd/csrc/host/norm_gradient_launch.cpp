// C-ABI entry point for the fused kernel-gradient contraction.
#include "host_common.hpp"
#include "../kernels/norm_gradient_mfma.hpp"

using namespace kmc_host;

namespace kmc_host {
hipError_t launch_norm_gradient(int norm_type, int o_tile, const kmc::NormGradientArgs &args, dim3 grid,
                                hipStream_t stream);
int64_t norm_gradient_f16_bytes(const kmc_norm_gradient_params *p);
hipError_t launch_norm_gradient_f16(const kmc_norm_gradient_params *p, bool a_vec, bool c_vec, bool e_vec, hipStream_t stream,
                                    bool *taken);
int64_t norm_gradient_l2_wide_bytes(const kmc_norm_gradient_params *p);
int launch_norm_gradient_l2_wide(const kmc_norm_gradient_params *p, hipStream_t stream, bool *taken);
}

namespace {

bool vec_ok(const void *ptr, int64_t s0, int64_t s1, int64_t s2, int flags)
{
    return !(flags & KMC_FLAG_FORCE_SCALAR_ACCESS) && aligned16(ptr) && s0 % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0;
}

}  // namespace

namespace {

int check(const kmc_norm_gradient_params *p)
{
    if (!p) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    if (p->norm_type < KMC_NORM_L1 || p->norm_type > KMC_NORM_P)
        return fail(KMC_ERR_INVALID_ARGUMENT, "norm_type %d is not a kmc_norm_type", p->norm_type);
    if (p->m < 0 || p->n < 0 || p->o < 0 || p->k < 0 || p->l < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative extent (m=%d n=%d o=%d k=%d l=%d)", p->m, p->n, p->o, p->k, p->l);
    if (p->m == 0 || p->n == 0 || p->o == 0 || p->l == 0) return KMC_OK;
    if (p->l > 65535) return fail(KMC_ERR_INVALID_ARGUMENT, "batch count %d exceeds 65535", p->l);
    if (!p->e || !p->d || (p->k > 0 && (!p->a || !p->b || !p->c)))
        return fail(KMC_ERR_INVALID_ARGUMENT, "null tensor pointer");
    if ((p->k > 1 && p->a_ld < p->m) || (p->n > 1 && p->b_ld < p->k) || (p->o > 1 && p->c_ld < p->k) ||
        (p->n > 1 && p->d_ld < p->m) || (p->n > 1 && p->e_ld_n < p->m))
        return fail(KMC_ERR_INVALID_ARGUMENT, "a leading dimension is smaller than the contiguous extent it spans");
    if (p->a_ld < 0 || p->b_ld < 0 || p->c_ld < 0 || p->d_ld < 0 || p->e_ld_n < 0 || p->e_ld_o < 0 || p->a_bs < 0 ||
        p->b_bs < 0 || p->c_bs < 0 || p->d_bs < 0 || p->e_bs < 0 || p->p_bs < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative stride");
    return KMC_OK;
}

}  // namespace

extern "C" int kmc_norm_gradient_workspace_bytes(const kmc_norm_gradient_params *p, int64_t *bytes)
{
    if (!bytes) return fail(KMC_ERR_INVALID_ARGUMENT, "bytes: null pointer");
    int status = check(p);
    if (status != KMC_OK) return status;
    if (p->m == 0 || p->n == 0 || p->o == 0 || p->l == 0) *bytes = 0;
    else *bytes = p->norm_type == KMC_NORM_L2 ? norm_gradient_l2_wide_bytes(p) : norm_gradient_f16_bytes(p);
    return KMC_OK;
}

extern "C" int kmc_norm_kernel_gradient(const kmc_norm_gradient_params *p, void *stream)
{
    int checked = check(p);
    if (checked != KMC_OK) return checked;
    if (p->m == 0 || p->n == 0 || p->o == 0 || p->l == 0) return KMC_OK;
    if (p->norm_type == KMC_NORM_L1 && p->workspace) {
        int ready = require_gfx950();
        if (ready != KMC_OK) return ready;
        bool taken = false;
        hipError_t e = launch_norm_gradient_f16(p, vec_ok(p->a, p->a_ld, p->a_bs, 0, p->flags), vec_ok(p->c, p->c_ld, p->c_bs, 0, p->flags),
                                                vec_ok(p->e, p->e_ld_n, p->e_ld_o, p->e_bs, p->flags), static_cast<hipStream_t>(stream),
                                                &taken);
        if (e != hipSuccess) return fail_hip(e, "norm_gradient_l1_f16 launches");
        if (taken) return KMC_OK;
    }
    if (p->norm_type == KMC_NORM_L2 && p->workspace && p->k > 0) {
        int ready = require_gfx950();
        if (ready != KMC_OK) return ready;
        bool taken = false;
        const int launched = launch_norm_gradient_l2_wide(p, static_cast<hipStream_t>(stream), &taken);
        if (launched != KMC_OK) return launched;
        if (taken) return KMC_OK;
    }

    // The outputs are cut into at most three runs, each with the kernel that suits its
    // width: whole groups of 32 (and a remainder of 25..31) on the matrix-core kernel with
    // 32 output columns, a remainder of 9..24 as 16 columns on the matrix-core kernel with
    // 16 plus, above 16, the rest on the vector-ALU kernel, which holds 1 to 6 or 8
    // accumulators per (m, n).  O = 17 therefore costs a 16-wide and a 1-wide launch
    // instead of one 32-wide launch that is half padding (18.5 -> 12.4 ms at M = K = 8192,
    // N = 512 for the L1 norm; O = 48: 36.6 -> 28.0 ms).
    struct Run { int begin, count, tile; };
    Run runs[3];
    int run_count = 0;
    {
        // the vector-ALU kernel exists for the widths 1..6 and 8 (7 accumulators per (m, n) measured
        // slower than 8 with one padded: 7.8 against 7.3 ms)
        auto small_tile = [](int o) { return o == 7 ? 8 : o; };
        int begin = 0, left = p->o;
        const int wide = left % 32 >= 25 ? left : left - left % 32;     // columns for the 32-wide kernel
        if (wide > 0) { runs[run_count++] = {begin, wide, 32}; begin += wide; left -= wide; }
        if (left >= 17 && p->norm_type == KMC_NORM_P) {
            // every run recomputes |d - b|^(p-1) with two transcendentals per (m, n, k): measured,
            // one padded 32-wide launch (24.5 ms at the benchmark shape) beats 16 + rest (25.6 .. 32 ms)
            runs[run_count++] = {begin, left, 32};
            left = 0;
        }
        if (left >= 9) { const int take = left < 16 ? left : 16; runs[run_count++] = {begin, take, 16}; begin += take; left -= take; }
        if (left > 0) runs[run_count++] = {begin, left, small_tile(left)};
    }

    int status = require_gfx950();
    if (status != KMC_OK) return status;
    for (int r = 0; r < run_count; r++) {
        const Run &run = runs[r];
        const bool matrix_core = run.tile >= 16;
        const int o_chunks = ceil_div(run.count, run.tile);
        const int64_t grid_z = static_cast<int64_t>(p->l) * o_chunks;
        const int tiles_m = ceil_div(p->m, matrix_core ? kmc::NGM_TILE_M : kmc::NG_TILE_M);
        const int tiles_n = ceil_div(p->n, matrix_core ? kmc::NGM_TILE_N : kmc::NG_TILE_N);
        if (grid_z > 65535 || tiles_n > 65535)
            return fail(KMC_ERR_INVALID_ARGUMENT, "grid too large (n tiles %d, batch x o chunks %lld; limit 65535)", tiles_n,
                        static_cast<long long>(grid_z));

        kmc::NormGradientArgs args;
        args.m = p->m; args.n = p->n; args.o = run.count; args.k = p->k; args.l = p->l;
        args.a = p->a; args.a_ld = p->a_ld; args.a_bs = p->a_bs;
        args.b = p->b; args.b_ld = p->b_ld; args.b_bs = p->b_bs;
        args.c = p->c ? p->c + static_cast<int64_t>(run.begin) * p->c_ld : p->c;
        args.c_ld = p->c_ld; args.c_bs = p->c_bs;
        args.d = p->d; args.d_ld = p->d_ld; args.d_bs = p->d_bs;
        args.e = p->e + static_cast<int64_t>(run.begin) * p->e_ld_o;
        args.e_ld_n = p->e_ld_n; args.e_ld_o = p->e_ld_o; args.e_bs = p->e_bs;
        args.p = p->p; args.p_bs = p->p_bs; args.p_value = p->p_value;
        args.o_chunks = o_chunks;
        args.a_vec = vec_ok(p->a, p->a_ld, p->a_bs, 0, p->flags);
        args.b_vec = vec_ok(p->b, p->b_ld, p->b_bs, 0, p->flags);
        args.c_vec = vec_ok(args.c, p->c_ld, p->c_bs, 0, p->flags);
        args.e_vec = vec_ok(args.e, p->e_ld_n, p->e_ld_o, p->e_bs, p->flags);

        const dim3 grid(tiles_m, tiles_n, static_cast<unsigned>(grid_z));
        hipError_t e = launch_norm_gradient(p->norm_type, run.tile, args, grid, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return fail_hip(e, "norm_kernel_gradient launch");
    }
    return KMC_OK;
}
