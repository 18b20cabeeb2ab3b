// Host side of the two-piece fp16 matrix-core path for large squared-difference problems
// (gram_f16_wide.hpp): when it applies, how the caller's workspace is divided, and the launches.
// One instantiation per kernel: the layout of an operand in memory is a run-time property of the
// two row kernels and does not reach the product kernel at all.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "../host/host_common.hpp"
#include "launch.hpp"
#include "gram_f16_wide.hpp"

namespace kmc_host {

namespace {

constexpr int64_t REGION_ALIGN = 256;

struct OperandRegions {
    int rows_pad, batches;
    int64_t pieces_bs;       // chunks per batch entry
    int64_t stats_bs;        // floats per batch entry, for the squares and for the magnitudes
    int64_t pieces, squares, magnitudes, unscale;   // byte offsets into the workspace
};

struct WideLayout {
    int slices, slices_per_range, ranges;
    int tiles_m, tiles_n, tiles_n_padded;
    OperandRegions a, b;
    int64_t bytes;
};

// Whether the route pays for its extra launches and its coarser tiles (a CU holds one workgroup of
// 256 x 256, so a few hundred tiles do not fill the chip as evenly as four times as many of
// 128 x 128).  From sweeps against the one-step kernel, one-step / wide time:
//   * over all tiles of the batch: K = 1024 1.09 at 144 tiles, 1.3 at 256, 1.6 from 1024 on; K = 256 0.99
//     at 576, 1.15 at 1024, 1.25 at 4096; K = 64 1.0 at 1024, 1.07 from 2304 on; K = 32 never above 1;
//   * the split of the operands is paid once per row and earned back once per tile the row meets, so
//     each batch entry needs tiles in both directions: at K = 1024, 64 entries of 2 x 2 tiles 0.74,
//     of 4 x 4 1.03, of 8 x 8 1.25, of 16 x 16 1.46; 118 x 4 tiles 1.26, 118 x 2 0.83, 391 x 2 0.84.
//     The rule asks tiles_m * tiles_n / (tiles_m + tiles_n) >= 2.5 (5 x 5, or 4 x 7, or 3 x 15);
//   * rows that pad the last tile are computed and thrown away: 8 entries of 1280 x 1280 1.24, of
//     1290 x 1290 (6 x 6 tiles, 30 % padding) 0.86.  The rule asks for at most 20 % padding.
// KERMAC_AMD_WIDE_MIN_TILES = t replaces the rule by "at least t tiles" (read on every call, so that
// a test can send small shapes down the route).
bool wide_pays(int64_t m, int64_t n, int64_t tiles_m, int64_t tiles_n, int64_t tiles, int k)
{
    const char *text = std::getenv("KERMAC_AMD_WIDE_MIN_TILES");
    const int forced = text ? std::atoi(text) : 0;
    if (forced > 0) return tiles >= forced && k >= 1;
    if (k < 64 || tiles < 128 || tiles * k < 147456) return false;
    if (2 * tiles_m * tiles_n < 5 * (tiles_m + tiles_n)) return false;
    return 5 * m * n >= 4 * (tiles_m * kmc::GW_TILE) * (tiles_n * kmc::GW_TILE);
}

int64_t place(int64_t &cursor, int64_t bytes)
{
    const int64_t at = cursor;
    cursor = (cursor + bytes + REGION_ALIGN - 1) / REGION_ALIGN * REGION_ALIGN;
    return at;
}

void place_operand(OperandRegions &r, int rows, bool broadcast, int l, const WideLayout &layout, int64_t &cursor)
{
    r.rows_pad = (rows + kmc::GW_TILE - 1) / kmc::GW_TILE * kmc::GW_TILE;
    r.batches = broadcast ? 1 : l;
    r.pieces_bs = static_cast<int64_t>(layout.slices + kmc::GW_EXTRA_SLICES) * kmc::GW_SEGMENTS * r.rows_pad;
    r.stats_bs = static_cast<int64_t>(layout.ranges) * r.rows_pad;
    r.pieces = place(cursor, r.batches * r.pieces_bs * 16);
    r.squares = place(cursor, r.batches * r.stats_bs * 4);
    r.magnitudes = place(cursor, r.batches * r.stats_bs * 4);
    r.unscale = place(cursor, static_cast<int64_t>(r.batches) * r.rows_pad * 4);
}

bool wide_layout(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, WideLayout *layout)
{
    if (!(p->flags & KMC_FLAG_L2_GRAM_BF16)) return false;
    if (p->inner_operator != KMC_OP_DIFF || p->inner_power != KMC_POW_SQUARE) return false;
    if (args.m < 1 || args.n < 1 || args.l < 1) return false;
    layout->tiles_m = (args.m + kmc::GW_TILE - 1) / kmc::GW_TILE;
    layout->tiles_n = (args.n + kmc::GW_TILE - 1) / kmc::GW_TILE;
    // a panel against itself: the tiles on and below the diagonal
    const int64_t tiles = args.symmetric ? static_cast<int64_t>(layout->tiles_m) * (layout->tiles_m + 1) / 2
                                         : static_cast<int64_t>(layout->tiles_m) * layout->tiles_n;
    if (!wide_pays(args.m, args.n, layout->tiles_m, layout->tiles_n, tiles * args.l, args.k)) return false;
    int padded = (layout->tiles_n + kmc::BK_XCDS - 1) / kmc::BK_XCDS * kmc::BK_XCDS;
    if ((padded - layout->tiles_n) * 8 > layout->tiles_n) padded = layout->tiles_n;
    if (static_cast<int64_t>(layout->tiles_m) * padded > 0x7fffffff) return false;
    layout->tiles_n_padded = padded;
    layout->slices = (args.k + kmc::BK_TILE_K - 1) / kmc::BK_TILE_K;
    // at most 8 ranges of K per row: enough workgroups for the row kernels, few partial sums
    layout->slices_per_range = layout->slices / 8 > 8 ? (layout->slices + 7) / 8 : 8;
    layout->ranges = (layout->slices + layout->slices_per_range - 1) / layout->slices_per_range;
    int64_t cursor = 0;
    // an operand that is the same for every batch entry is split once, unless the centre differs
    const bool one_centre = !args.centre || args.centre_bs == 0;
    place_operand(layout->a, args.m, args.a_bs == 0 && one_centre, args.l, *layout, cursor);
    if (args.symmetric) layout->b = layout->a;      // one panel, split once
    else place_operand(layout->b, args.n, args.b_bs == 0 && one_centre, args.l, *layout, cursor);
    layout->bytes = cursor;
    return true;
}

kmc::GramRowsArgs rows_args(const float *x, int64_t ld, int64_t bs, int rows, int majorness, bool scalar_only,
                            const kmc::BuildKernelArgs &args, const WideLayout &layout, const OperandRegions &r, char *workspace)
{
    kmc::GramRowsArgs rows_of = {};
    rows_of.x = x; rows_of.ld = ld; rows_of.bs = bs;
    rows_of.rows = rows; rows_of.k = args.k;
    rows_of.row_major = majorness == KMC_ROW_MAJOR;
    rows_of.vec = rows_of.row_major && !scalar_only && aligned16(x) && ld % 4 == 0 && bs % 4 == 0;
    rows_of.centre = args.centre; rows_of.centre_bs = args.centre_bs;
    rows_of.pieces = reinterpret_cast<kmc::gram_chunk *>(workspace + r.pieces); rows_of.pieces_bs = r.pieces_bs;
    rows_of.squares = reinterpret_cast<float *>(workspace + r.squares);
    rows_of.magnitudes = reinterpret_cast<float *>(workspace + r.magnitudes);
    rows_of.unscale = reinterpret_cast<float *>(workspace + r.unscale);
    rows_of.stats_bs = r.stats_bs; rows_of.unscale_bs = r.rows_pad;
    rows_of.rows_pad = r.rows_pad; rows_of.slices = layout.slices;
    rows_of.slices_per_range = layout.slices_per_range; rows_of.ranges = layout.ranges;
    return rows_of;
}

}  // namespace

// Statistics and split of one operand (also used by the gradient's fp16 route).
hipError_t launch_gram_rows(const kmc::GramRowsArgs &rows_of, int batches, hipStream_t stream)
{
    const dim3 grid(rows_of.rows_pad / kmc::GW_ROW_THREADS, rows_of.ranges, batches);
    hipError_t status = launch(kmc::gram_row_stats<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, rows_of);
    if (status != hipSuccess) return status;
    return launch(kmc::gram_f16_split<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, rows_of);
}

// Bytes of workspace the path needs for this problem; 0 when it does not apply.
int64_t gram_f16_wide_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args)
{
    WideLayout layout;
    return wide_layout(p, args, &layout) ? layout.bytes : 0;
}

// Row statistics and split of both operands, then the product kernel.  `*taken` says whether the
// path applied (and the launches were made); if not, nothing was launched.
hipError_t launch_gram_f16_wide(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *taken)
{
    *taken = false;
    WideLayout layout;
    if (!p->gram_workspace || !wide_layout(p, args, &layout) || p->gram_workspace_bytes < layout.bytes ||
        (reinterpret_cast<uintptr_t>(p->gram_workspace) & (REGION_ALIGN - 1)) != 0)
        return hipSuccess;
    char *workspace = static_cast<char *>(p->gram_workspace);
    const bool scalar_only = (p->flags & KMC_FLAG_FORCE_SCALAR_ACCESS) != 0;
    const kmc::GramRowsArgs rows_a = rows_args(args.a, args.a_ld, args.a_bs, args.m, p->a_majorness, scalar_only, args, layout, layout.a, workspace);
    const kmc::GramRowsArgs rows_b = rows_args(args.b, args.b_ld, args.b_bs, args.n, p->b_majorness, scalar_only, args, layout, layout.b, workspace);
    // the region of a lies first in the workspace and its size does not depend on b
    hipError_t status = (p->flags & KMC_FLAG_GRAM_A_KEPT) ? hipSuccess : launch_gram_rows(rows_a, layout.a.batches, stream);
    if (status != hipSuccess) return status;
    if (!args.symmetric) {
        status = launch_gram_rows(rows_b, layout.b.batches, stream);
        if (status != hipSuccess) return status;
    }

    kmc::GramWideArgs wide = {};
    wide.kernel = args;
    wide.pieces_a = rows_a.pieces; wide.pieces_b = rows_b.pieces;
    wide.pieces_a_bs = layout.a.batches > 1 ? layout.a.pieces_bs : 0;
    wide.pieces_b_bs = layout.b.batches > 1 ? layout.b.pieces_bs : 0;
    wide.squares_a = rows_a.squares; wide.squares_b = rows_b.squares;
    wide.stats_a_bs = layout.a.batches > 1 ? layout.a.stats_bs : 0;
    wide.stats_b_bs = layout.b.batches > 1 ? layout.b.stats_bs : 0;
    wide.unscale_a = rows_a.unscale; wide.unscale_b = rows_b.unscale;
    wide.unscale_a_bs = layout.a.batches > 1 ? layout.a.rows_pad : 0;
    wide.unscale_b_bs = layout.b.batches > 1 ? layout.b.rows_pad : 0;
    wide.rows_pad_a = layout.a.rows_pad; wide.rows_pad_b = layout.b.rows_pad;
    wide.slices = layout.slices; wide.ranges = layout.ranges;
    wide.wide_tiles_m = layout.tiles_m; wide.wide_tiles_n = layout.tiles_n; wide.wide_tiles_n_padded = layout.tiles_n_padded;
    if (args.symmetric) {
        const dim3 grid(static_cast<unsigned>(layout.tiles_m) * (layout.tiles_m + 1) / 2, args.l, 1);
        status = launch(kmc::gram_f16_wide<true>, grid, dim3(kmc::GW_THREADS), stream, wide);
    } else {
        const dim3 grid(static_cast<unsigned>(layout.tiles_m) * layout.tiles_n_padded, args.l, 1);
        status = launch(kmc::gram_f16_wide<false>, grid, dim3(kmc::GW_THREADS), stream, wide);
    }
    if (status == hipSuccess) *taken = true;
    return status;
}

}  // namespace kmc_host
