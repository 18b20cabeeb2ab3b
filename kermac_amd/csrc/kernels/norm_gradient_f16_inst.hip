// Host side of the L1 kernel gradient on the fp16 matrix instruction (norm_gradient_f16.hpp): when
// it applies, how the caller's workspace is divided, and the launches: row statistics and split of
// A (rows m) and of C (rows o) by the kernels of gram_f16_wide.hpp, a padded copy of B, the
// contraction.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "../host/host_common.hpp"
#include "../host/dispatch_rules.hpp"
#include "launch.hpp"
#include "norm_gradient_f16.hpp"

namespace kmc_host {

namespace {

constexpr int64_t REGION_ALIGN = 256;

struct RowsRegions {
    int rows_pad, batches;
    int64_t pieces_bs, stats_bs;
    int64_t pieces, squares, magnitudes, unscale;     // byte offsets into the workspace
};

struct GradientLayout {
    int slices, slices_alloc, slices_per_range, ranges, steps;
    int n_pad, k_pad, b_batches;
    RowsRegions a, c;
    int64_t b_padded, b_padded_bs;
    int64_t bytes;
};

int64_t place(int64_t &cursor, int64_t bytes)
{
    const int64_t at = cursor;
    cursor = (cursor + bytes + REGION_ALIGN - 1) / REGION_ALIGN * REGION_ALIGN;
    return at;
}

void place_rows(RowsRegions &r, int rows, int batches, const GradientLayout &layout, int64_t &cursor)
{
    r.rows_pad = (rows + kmc::GW_TILE - 1) / kmc::GW_TILE * kmc::GW_TILE;
    r.batches = batches;
    r.pieces_bs = static_cast<int64_t>(layout.slices_alloc) * kmc::GW_SEGMENTS * r.rows_pad;
    r.stats_bs = static_cast<int64_t>(layout.ranges) * r.rows_pad;
    r.pieces = place(cursor, r.batches * r.pieces_bs * 16);
    r.squares = place(cursor, r.batches * r.stats_bs * 4);
    r.magnitudes = place(cursor, r.batches * r.stats_bs * 4);
    r.unscale = place(cursor, static_cast<int64_t>(r.batches) * r.rows_pad * 4);
}

// The route pays where the fp32 kernels are bound by their matrix or vector instructions: enough
// terms to carry the five extra launches, and more than two outputs (its cost does not fall below
// that of 16 outputs; the vector kernel for one or two is cheaper).  From sweeps, fp32 / fp16 time:
// O = 16 at 3.4e10 terms 2.5, 1.1e9 1.8, 5.4e8 1.1 .. 1.4, 2.7e8 0.8 .. 1.1, 1.3e8 0.66; at 3.4e10
// terms O = 1 0.73, O = 2 0.93, O = 3 1.21, O = 4 1.31, O = 8 2.1, O = 17 1.7, O = 48 2.6; with few
// outputs the fp32 kernels are cheaper by nearly that factor and the route is not (16 results per
// tile whatever O), so the terms are asked for in proportion: 4e8 at 16 outputs, 1.6e9 at 4.  Its
// tiles hold 32 columns of the result: N = 8 0.90, N = 16 0.86, N = 32 1.37, N = 33 1.49.
// KERMAC_AMD_GRADIENT_F16_MIN_TERMS replaces the conditions by a number of terms (read on every
// call, so that a test can send small shapes down the route).
bool f16_pays(const kmc_norm_gradient_params *p)
{
    const char *text = std::getenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS");
    const double forced = text ? std::atof(text) : 0.0;
    const double terms = static_cast<double>(p->m) * p->n * p->k * p->l;
    if (forced > 0.0) return terms >= forced;
    // more than 16 outputs: the wider tiles of the route share the sign work between blocks of outputs, while the
    // fp32 kernels go to their 32-column tiles (O = 32: 98 against 75 us at 1.7e7 terms, 187 against 128 at 2.7e8;
    // O = 128: 101 against 70 and 588 against 206)
    namespace r = kmc_rules;
    if (p->o > 16) return p->n >= r::GRADIENT_F16_MIN_N && terms >= static_cast<double>(r::GRADIENT_F16_MANY_OUTPUTS_MIN_TERMS);
    return p->o >= r::GRADIENT_F16_MIN_OUTPUTS && p->n >= r::GRADIENT_F16_MIN_N &&
           terms * p->o >= static_cast<double>(r::GRADIENT_F16_MIN_TERMS_TIMES_OUTPUTS);
}

bool gradient_layout(const kmc_norm_gradient_params *p, GradientLayout *layout)
{
    if (p->norm_type != KMC_NORM_L1 || p->m < 1 || p->n < 1 || p->o < 1 || p->k < 1 || p->l < 1) return false;
    if (!f16_pays(p)) return false;
    layout->slices = (p->k + kmc::BK_TILE_K - 1) / kmc::BK_TILE_K;
    layout->steps = (p->k + kmc::NGF_STEP_K - 1) / kmc::NGF_STEP_K;
    layout->slices_alloc = 2 * (layout->steps + kmc::NGF_AHEAD);
    layout->slices_per_range = layout->slices / 8 > 8 ? (layout->slices + 7) / 8 : 8;
    layout->ranges = (layout->slices + layout->slices_per_range - 1) / layout->slices_per_range;
    layout->n_pad = (p->n + kmc::NGF_N_PAD - 1) / kmc::NGF_N_PAD * kmc::NGF_N_PAD;
    layout->k_pad = kmc::NGF_STEP_K * (layout->steps + kmc::NGF_AHEAD);
    int64_t cursor = 0;
    place_rows(layout->a, p->m, p->a_bs == 0 ? 1 : p->l, *layout, cursor);
    place_rows(layout->c, p->o, p->c_bs == 0 ? 1 : p->l, *layout, cursor);
    layout->b_batches = p->b_bs == 0 ? 1 : p->l;
    layout->b_padded_bs = static_cast<int64_t>(layout->n_pad) * layout->k_pad;
    layout->b_padded = place(cursor, layout->b_batches * layout->b_padded_bs * 4);
    layout->bytes = cursor;
    // blockIdx.z = batch entry x chunk of outputs; blockIdx.y = one padded row n for gradient_pad_b (the
    // largest grid.y of the route; the contraction's tiles of 8, 16 or 32 n need fewer)
    const int64_t grid_z = static_cast<int64_t>(p->l) * (p->o / 64 + 1);
    if (grid_z > 65535 || layout->n_pad > 65535) return false;
    return true;
}

kmc::GramRowsArgs rows_args(const float *x, int64_t ld, int64_t bs, int rows, bool row_major, bool vec, int k,
                            const GradientLayout &layout, const RowsRegions &r, char *workspace)
{
    kmc::GramRowsArgs rows_of = {};
    rows_of.x = x; rows_of.ld = ld; rows_of.bs = bs;
    rows_of.rows = rows; rows_of.k = k;
    rows_of.row_major = row_major; rows_of.vec = row_major && vec;
    rows_of.pieces = reinterpret_cast<kmc::gram_chunk *>(workspace + r.pieces); rows_of.pieces_bs = r.pieces_bs;
    rows_of.squares = reinterpret_cast<float *>(workspace + r.squares);
    rows_of.magnitudes = reinterpret_cast<float *>(workspace + r.magnitudes);
    rows_of.unscale = reinterpret_cast<float *>(workspace + r.unscale);
    rows_of.stats_bs = r.stats_bs; rows_of.unscale_bs = r.rows_pad;
    rows_of.rows_pad = r.rows_pad; rows_of.slices = layout.slices;
    rows_of.slices_per_range = layout.slices_per_range; rows_of.ranges = layout.ranges;
    rows_of.zero_slices = 2 * layout.steps - layout.slices;      // the walk takes two slices per step
    return rows_of;
}

}  // namespace

hipError_t launch_gram_rows_pair(const kmc::GramRowsArgs &first, int first_batches, const kmc::GramRowsArgs &second, int second_batches,
                                 hipStream_t stream);     // gram_f16_wide_inst.hip

int64_t norm_gradient_f16_bytes(const kmc_norm_gradient_params *p)
{
    GradientLayout layout;
    return gradient_layout(p, &layout) ? layout.bytes : 0;
}

// `*taken` says whether the route applied (and the launches were made); if not, nothing was launched.
hipError_t launch_norm_gradient_f16(const kmc_norm_gradient_params *p, bool a_vec, bool c_vec, bool e_vec, hipStream_t stream,
                                    bool *taken)
{
    *taken = false;
    GradientLayout layout;
    if (!p->workspace || !gradient_layout(p, &layout) || p->workspace_bytes < layout.bytes ||
        (reinterpret_cast<uintptr_t>(p->workspace) & (REGION_ALIGN - 1)) != 0)
        return hipSuccess;
    char *workspace = static_cast<char *>(p->workspace);
    (void)a_vec;
    const kmc::GramRowsArgs rows_a = rows_args(p->a, p->a_ld, p->a_bs, p->m, false, false, p->k, layout, layout.a, workspace);
    const kmc::GramRowsArgs rows_c = rows_args(p->c, p->c_ld, p->c_bs, p->o, true, c_vec, p->k, layout, layout.c, workspace);
    hipError_t status = launch_gram_rows_pair(rows_a, layout.a.batches, rows_c, layout.c.batches, stream);
    if (status != hipSuccess) return status;

    kmc::GradientPadArgs pad = {};
    pad.b = p->b; pad.b_ld = p->b_ld; pad.b_bs = p->b_bs;
    pad.padded = reinterpret_cast<float *>(workspace + layout.b_padded); pad.padded_bs = layout.b_padded_bs;
    pad.n = p->n; pad.k = p->k; pad.n_pad = layout.n_pad; pad.k_pad = layout.k_pad;
    status = launch(kmc::gradient_pad_b, dim3((layout.k_pad / 4 + 255) / 256, layout.n_pad, layout.b_batches), dim3(256), stream, pad);
    if (status != hipSuccess) return status;

    kmc::NormGradientF16Args args = {};
    args.g.m = p->m; args.g.n = p->n; args.g.o = p->o; args.g.k = p->k; args.g.l = p->l;
    args.g.d = p->d; args.g.d_ld = p->d_ld; args.g.d_bs = p->d_bs;
    args.g.e = p->e; args.g.e_ld_n = p->e_ld_n; args.g.e_ld_o = p->e_ld_o; args.g.e_bs = p->e_bs;
    args.g.e_vec = e_vec;
    args.pieces_a = rows_a.pieces; args.pieces_c = rows_c.pieces;
    args.pieces_a_bs = layout.a.batches > 1 ? layout.a.pieces_bs : 0;
    args.pieces_c_bs = layout.c.batches > 1 ? layout.c.pieces_bs : 0;
    args.unscale_a = rows_a.unscale; args.unscale_c = rows_c.unscale;
    args.unscale_a_bs = layout.a.batches > 1 ? layout.a.rows_pad : 0;
    args.unscale_c_bs = layout.c.batches > 1 ? layout.c.rows_pad : 0;
    args.b_padded = pad.padded;
    args.b_padded_bs = layout.b_batches > 1 ? layout.b_padded_bs : 0;
    args.rows_pad_a = layout.a.rows_pad; args.rows_pad_c = layout.c.rows_pad;
    args.k_pad = layout.k_pad; args.steps = layout.steps;
    // Outputs in chunks of 64 on the 8 n x 64 o tile while more than 32 are left, then one chunk of 32 on the
    // 16 n x 32 o tile for 17 to 32 of them, or the 32 n x 16 o tile for up to 16.
    int wide_chunks = p->o / 64;
    int left = p->o % 64;
    if (left > 32) { wide_chunks += 1; left = 0; }
    const unsigned tiles_m = (p->m + kmc::NGF_TILE_M - 1) / kmc::NGF_TILE_M;
    auto run = [&](auto blocks, int o_begin, int chunks) {
        using Tile = kmc::GradientF16Tile<decltype(blocks)::value>;
        args.o_begin = o_begin;
        args.g.o_chunks = chunks;
        const dim3 grid(tiles_m, (p->n + Tile::TILE_N - 1) / Tile::TILE_N, static_cast<unsigned>(p->l) * chunks);
        return launch(kmc::norm_gradient_l1_f16<decltype(blocks)::value>, grid, dim3(kmc::NGF_THREADS), stream, args);
    };
    if (wide_chunks) {
        status = run(std::integral_constant<int, 4>{}, 0, wide_chunks);
        if (status != hipSuccess) return status;
    }
    if (left > 16) status = run(std::integral_constant<int, 2>{}, p->o - left, 1);
    else if (left > 0) status = run(std::integral_constant<int, 1>{}, p->o - left, 1);
    if (status == hipSuccess) *taken = true;
    return status;
}

}  // namespace kmc_host
