// Host side of the two-piece fp16 matrix-core path for large squared-difference problems
// (gram_f16_wide.hpp): when it applies, how the caller's workspace is divided, and the launches.
// One instantiation per kernel: the layout of an operand in memory is a run-time property of the
// two row kernels and does not reach the product kernel at all.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>

#include "../host/host_common.hpp"
#include "../host/dispatch_rules.hpp"
#include "launch.hpp"
#include "gram_f16_wide.hpp"
#include "norm_gradient_l2_wide.hpp"

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
    int64_t sample;         // byte offset of the words of gram_probe_operands
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
// Sums of products have no one-step matrix-core kernel to fall back to: the alternative is the direct
// kernel, which the route beats much earlier (direct / route time: 64 tiles 1.04 .. 1.42 at K = 1024,
// 0.82 .. 1.04 at K = 512; 256 tiles 1.25 at K = 256, 0.86 at K = 128; 1024 tiles 1.17 .. 1.35 at K = 128,
// 0.91 .. 1.02 at K = 64; 64 batch entries of 2 x 2 tiles 1.5, 118 x 2 tiles 1.9).  From K = 256 on it is
// taken from 32 tiles and tiles * k = 24576 on whatever the padding (8 entries of 512 x 512 x 784 1.3 .. 1.4, at
// K = 3072 1.7 .. 1.9; 4 of 1000 x 1000 x 784 1.7; 144 tiles at K = 256 1.2 .. 1.3; 300 x 30000, 41 % of the tiles
// padding, 1.1 .. 1.2 at K = 256 and 1.7 .. 1.9 beyond; at K = 256 with 64 tiles 0.8 .. 0.9), but a single problem
// only from 64 tiles on: the direct path cuts such a call over k (1500 x 1500, 36 tiles: 0.77 .. 0.84).
//
// Operands with k contiguous (row-major, as torch allocates them): the one-step kernels stage such operands
// more slowly, the route splits them once and walks pieces whose layout is its own, so it pays much earlier
// and whatever the shape of a batch entry (one-step / route time: 64 tiles 1.2 at K = 784, 1.5 at K = 3072, also
// as 16 entries of 2 x 2 tiles with a third of the tiles padding; 144 tiles 1.1 at K = 256, 1.8 at K = 784;
// 2 x 118 tiles 1.07 at K = 256, 1.3 at K = 784; 36 tiles 0.9 / 1.2; 32 tiles as 8 entries of 2 x 2 0.75 / 0.8;
// K = 128 never above 1).  Not for a dimension that half a tile holds, where the 128 x 128 tiles of the
// one-step kernels waste half as much (100 x 50000: 0.87 at K = 784, 4 entries 0.73; 128 x 20000 0.8).
bool wide_pays(int64_t m, int64_t n, int64_t tiles_m, int64_t tiles_n, int64_t tiles, int k, bool products, bool k_contiguous,
               bool batched)
{
    const char *text = std::getenv("KERMAC_AMD_WIDE_MIN_TILES");
    const int forced = text ? std::atoi(text) : 0;
    if (forced > 0) return tiles >= forced && k >= 1;
    namespace r = kmc_rules;
    if (k_contiguous && !products && k >= r::WIDE_K_CONTIGUOUS_MIN_K && tiles >= r::WIDE_K_CONTIGUOUS_MIN_TILES &&
        tiles * k >= r::WIDE_K_CONTIGUOUS_MIN_TILES_TIMES_K && m >= r::WIDE_K_CONTIGUOUS_MIN_ROWS && n >= r::WIDE_K_CONTIGUOUS_MIN_ROWS)
        return true;
    const bool little_padding = 100 * m * n >= (100 - r::WIDE_MAX_PADDING_PERCENT) * (tiles_m * kmc::GW_TILE) * (tiles_n * kmc::GW_TILE);
    if (products && k >= r::DOT_LONG_K && tiles * k >= r::DOT_LONG_MIN_TILES_TIMES_K &&
        tiles >= (batched ? r::DOT_LONG_MIN_TILES_BATCHED : r::DOT_LONG_MIN_TILES_SINGLE))
        return true;
    if (products) return k >= r::DOT_MIN_K && tiles >= r::DOT_MIN_TILES && tiles * k >= r::DOT_MIN_TILES_TIMES_K && little_padding;
    // (from 768 tiles on the route is as fast as the one-step kernel also for the shortest contractions
    // it takes, 8192 x 8192 x 64 180 us against 187, and ahead of the direct kernel, 236)
    if (k < r::WIDE_MIN_K || tiles < r::WIDE_MIN_TILES || (tiles * k < r::WIDE_MIN_TILES_TIMES_K && tiles < r::WIDE_TILES_FOR_ANY_K)) return false;
    if (2 * tiles_m * tiles_n < r::WIDE_MIN_TILES_PER_SIDE_X2 * (tiles_m + tiles_n)) return false;
    return little_padding;
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

// Grid, slices and the regions of both operands in the workspace; tiles_m and tiles_n are set.
bool place_wide(int m, int n, int k, int l, bool a_once, bool b_once, bool symmetric, WideLayout *layout)
{
    int padded = (layout->tiles_n + kmc::BK_XCDS - 1) / kmc::BK_XCDS * kmc::BK_XCDS;
    if ((padded - layout->tiles_n) * 8 > layout->tiles_n) padded = layout->tiles_n;
    if (static_cast<int64_t>(layout->tiles_m) * padded > 0x7fffffff) return false;
    layout->tiles_n_padded = padded;
    layout->slices = (k + kmc::BK_TILE_K - 1) / kmc::BK_TILE_K;
    // at most 8 ranges of K per row: enough workgroups for the row kernels, few partial sums
    layout->slices_per_range = layout->slices / 8 > 8 ? (layout->slices + 7) / 8 : 8;
    layout->ranges = (layout->slices + layout->slices_per_range - 1) / layout->slices_per_range;
    if (layout->ranges > kmc::GW_MAX_RANGES) return false;       // 9 at most by the two lines above
    int64_t cursor = 0;
    place_operand(layout->a, m, a_once, l, *layout, cursor);
    if (symmetric) layout->b = layout->a;      // one panel, split once
    else place_operand(layout->b, n, b_once, l, *layout, cursor);
    layout->sample = place(cursor, kmc::BK_SAMPLE_BYTES);
    layout->bytes = cursor;
    return true;
}

bool wide_layout(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, WideLayout *layout)
{
    const bool squared_differences = (p->flags & KMC_FLAG_L2_GRAM_BF16) && p->inner_operator == KMC_OP_DIFF && p->inner_power == KMC_POW_SQUARE;
    const bool products = (p->flags & KMC_FLAG_DOT_PIECES) && p->inner_operator == KMC_OP_DOT && p->inner_power == KMC_POW_NOOP;
    if (!squared_differences && !products) return false;
    if (args.m < 1 || args.n < 1 || args.l < 1) return false;
    layout->tiles_m = (args.m + kmc::GW_TILE - 1) / kmc::GW_TILE;
    layout->tiles_n = (args.n + kmc::GW_TILE - 1) / kmc::GW_TILE;
    // a panel against itself: the tiles on and below the diagonal
    const int64_t tiles = args.symmetric ? static_cast<int64_t>(layout->tiles_m) * (layout->tiles_m + 1) / 2
                                         : static_cast<int64_t>(layout->tiles_m) * layout->tiles_n;
    const bool k_contiguous = p->a_majorness == KMC_ROW_MAJOR && p->b_majorness == KMC_ROW_MAJOR;
    const bool asked_for = (p->flags & KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE) && args.k >= 1;
    if (!asked_for && !wide_pays(args.m, args.n, layout->tiles_m, layout->tiles_n, tiles * args.l, args.k, products, k_contiguous, args.l > 1)) return false;
    // an operand that is the same for every batch entry is split once, unless the centre differs
    // (products have no centre: the caller's parameter block carries none into `args`)
    const bool one_centre = products || !args.centre || args.centre_bs == 0;
    return place_wide(args.m, args.n, args.k, args.l, args.a_bs == 0 && one_centre, args.b_bs == 0 && one_centre, args.symmetric, layout);
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

// What the split of `a` in a workspace was made from, kept on the host per workspace address: a call with
// KMC_FLAG_GRAM_A_KEPT skips the split only when this record says that the previous split through this
// workspace was of the same operand, shape, centre and layout; anything else (another operand, a call
// that did not take this route in between and left no record, a workspace seen for the first time)
// makes the split again.  What the host cannot see is whether the memory itself was overwritten since.
struct SplitRecord {
    const float *a; int64_t ld, bs; int majorness, m, k, l, slices, rows_pad;
    const float *centre; int64_t centre_bs;
};

std::mutex split_records_mutex;
std::unordered_map<const void *, SplitRecord> split_records;

SplitRecord record_of(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, const WideLayout &layout)
{
    SplitRecord record;
    std::memset(&record, 0, sizeof record);          // padding too: the records are compared as bytes
    record.a = p->a; record.ld = p->a_ld; record.bs = p->a_bs; record.majorness = p->a_majorness;
    record.m = p->m; record.k = p->k; record.l = layout.a.batches; record.slices = layout.slices; record.rows_pad = layout.a.rows_pad;
    record.centre = args.centre; record.centre_bs = args.centre_bs;
    return record;
}

// true: the split of `a` in this workspace is the one this call needs; either way the record is this call's afterwards
bool split_of_a_is_kept(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, const WideLayout &layout)
{
    const SplitRecord wanted = record_of(p, args, layout);
    std::lock_guard<std::mutex> lock(split_records_mutex);
    auto found = split_records.find(p->gram_workspace);
    const bool kept = (p->flags & KMC_FLAG_GRAM_A_KEPT) && found != split_records.end() &&
                      std::memcmp(&found->second, &wanted, sizeof wanted) == 0;
    if (split_records.size() > 4096) split_records.clear();      // addresses of freed workspaces pile up otherwise
    split_records[p->gram_workspace] = wanted;
    return kept;
}

}  // namespace

// A route other than this one is about to write into `workspace`: whatever split it held is gone.
void forget_split_in(const void *workspace)
{
    std::lock_guard<std::mutex> lock(split_records_mutex);
    split_records.erase(workspace);
}

// Statistics and split of one operand (also used by the gradient's fp16 route).
hipError_t launch_gram_probe(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, unsigned *sample, hipStream_t stream);   // gram_probe.hip

hipError_t launch_gram_rows(const kmc::GramRowsArgs &rows_of, int batches, hipStream_t stream)
{
    const dim3 grid(rows_of.rows_pad / kmc::GW_ROW_THREADS, rows_of.ranges, batches);
    hipError_t status = launch(kmc::gram_row_stats<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, rows_of);
    if (status != hipSuccess) return status;
    return launch(kmc::gram_f16_split<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, rows_of);
}

// The same for both operands of a call, in two launches instead of four.
hipError_t launch_gram_rows_pair(const kmc::GramRowsArgs &first, int first_batches, const kmc::GramRowsArgs &second, int second_batches,
                                 hipStream_t stream)
{
    if (first.ranges != second.ranges) {
        hipError_t status = launch_gram_rows(first, first_batches, stream);
        return status != hipSuccess ? status : launch_gram_rows(second, second_batches, stream);
    }
    kmc::GramRowsPair pair;
    pair.first = first; pair.second = second;
    pair.first_blocks = first.rows_pad / kmc::GW_ROW_THREADS;
    pair.first_batches = first_batches; pair.second_batches = second_batches;
    const dim3 grid(pair.first_blocks + second.rows_pad / kmc::GW_ROW_THREADS, first.ranges, first_batches > second_batches ? first_batches : second_batches);
    hipError_t status = launch(kmc::gram_row_stats_pair<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, pair);
    if (status != hipSuccess) return status;
    return launch(kmc::gram_f16_split_pair<0>, grid, dim3(kmc::GW_ROW_THREADS), stream, pair);
}

// Bytes of workspace the path needs for this problem; 0 when it does not apply.
int64_t gram_f16_wide_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args)
{
    WideLayout layout;
    return wide_layout(p, args, &layout) ? layout.bytes : 0;
}

// Row statistics and split of both operands, then the product kernel.  `*taken` says whether the
// path applied (and the launches were made); if not, nothing was launched.
hipError_t launch_gram_f16_wide(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *taken,
                                const unsigned **sample_taken)
{
    *taken = false;
    if (sample_taken) *sample_taken = nullptr;
    WideLayout layout;
    if (!p->gram_workspace || !wide_layout(p, args, &layout) || p->gram_workspace_bytes < layout.bytes ||
        (reinterpret_cast<uintptr_t>(p->gram_workspace) & (REGION_ALIGN - 1)) != 0)
        return hipSuccess;
    char *workspace = static_cast<char *>(p->gram_workspace);
    const bool scalar_only = (p->flags & KMC_FLAG_FORCE_SCALAR_ACCESS) != 0;
    const kmc::GramRowsArgs rows_a = rows_args(args.a, args.a_ld, args.a_bs, args.m, p->a_majorness, scalar_only, args, layout, layout.a, workspace);
    const kmc::GramRowsArgs rows_b = rows_args(args.b, args.b_ld, args.b_bs, args.n, p->b_majorness, scalar_only, args, layout, layout.b, workspace);
    // the region of a lies first in the workspace and its size does not depend on b
    const bool a_is_kept = split_of_a_is_kept(p, args, layout);
    hipError_t status = hipSuccess;
    if (!a_is_kept && !args.symmetric) {
        status = launch_gram_rows_pair(rows_a, layout.a.batches, rows_b, layout.b.batches, stream);
    } else {
        if (!a_is_kept) status = launch_gram_rows(rows_a, layout.a.batches, stream);
        if (status == hipSuccess && !args.symmetric) status = launch_gram_rows(rows_b, layout.b.batches, stream);
    }
    if (status != hipSuccess) return status;

    kmc::GramWideArgs wide = {};
    wide.kernel = args;
    // The caller's trust rule grows with sqrt(k) (the error of a sum of k terms against the norms) and
    // passes 1 near k = 18000, where it would send every part to the repair launch -- whose own
    // fp32 sum over k is no better by then (measured at k = 20000 .. 200000: this walk, which rounds once
    // per 16 k, 4e-7 .. 2e-6 of d for points as far apart as their norms, the direct kernel 5e-6 .. 4e-5).
    // With a product worth half the norms the two are equally good, so that is where the rule stops.
    if (wide.kernel.gram_trust > 0.5f) wide.kernel.gram_trust = 0.5f;
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
    const bool products = p->inner_operator == KMC_OP_DOT;
    // Squared differences: a sample of the result first, so that data the trust rule would reject wholesale
    // (sets of near-duplicates) costs the direct kernel's time and little more, instead of both.
    // KMC_FLAG_NO_PROBE leaves it out.
    if (!products && !(p->flags & KMC_FLAG_NO_PROBE)) {
        unsigned *sample = reinterpret_cast<unsigned *>(workspace + layout.sample);
        status = launch_gram_probe(p, wide.kernel, sample, stream);
        if (status != hipSuccess) return status;
        wide.kernel.sample = sample;
        if (sample_taken) *sample_taken = sample;
    }
    if (args.symmetric) {
        const dim3 grid(static_cast<unsigned>(layout.tiles_m) * (layout.tiles_m + 1) / 2, args.l, 1);
        status = products ? launch(kmc::gram_f16_wide<true, kmc::GW_EPILOGUE_DOT>, grid, dim3(kmc::GW_THREADS), stream, wide)
                          : launch(kmc::gram_f16_wide<true>, grid, dim3(kmc::GW_THREADS), stream, wide);
    } else {
        const dim3 grid(static_cast<unsigned>(layout.tiles_m) * layout.tiles_n_padded, args.l, 1);
        status = products ? launch(kmc::gram_f16_wide<false, kmc::GW_EPILOGUE_DOT>, grid, dim3(kmc::GW_THREADS), stream, wide)
                          : launch(kmc::gram_f16_wide<false>, grid, dim3(kmc::GW_THREADS), stream, wide);
    }
    if (status == hipSuccess) *taken = true;
    return status;
}

// ---- the gradient of the L2 norm as one product of pieces (norm_gradient_l2_wide.hpp) ----

namespace {

struct GradientL2Layout {
    WideLayout wide;                 // a: the columns m of a; b: the rows (o, n) of the products
    int products_ld;
    int g_parts;                     // ranges of k that g is summed in (partial products, then their sum)
    int64_t products, shift, c_transposed, g, g_partial;      // byte offsets behind the regions of `wide`
    int64_t bytes;
};

// The route pays where a model of both times says so by 15 %, in microseconds, fitted to sweeps:
//   fp32 kernels   30 + terms * t(o) with terms = m n k l and t(o) = 0.077, 0.10, 0.126, 0.137 ps for 1 .. 4
//                  outputs, 0.028 o up to 8 (vector kernels), 0.27 up to 16, 0.56 up to 32, 0.0175 o beyond
//                  (matrix-core kernels: a run of outputs costs what its 16 or 32 columns cost);
//   this route     200 + 1.5e-6 (o n + m) k l for the products and the two splits, and for the walk
//                  6.3e-9 per multiply-add of the padded tiles (1.7 us per 256 x 256 x 16 step of a CU with the
//                  chip full) but not less than 0.056 k (a CU alone walks a step in 0.9 us).
// Examples (fp32 / this route, measured): 8192 x 512 x 16 x 8192 2.7; o = 1 .. 8 there 2.8 .. 4.0; n = 64 1.75,
// n = 32 0.96, n = 8 0.81; m = 1024 1.55, m = 512 0.86; k = 512 1.35, k = 256 0.92, k = 64 0.40;
// 10000 x 1000 x 10 x 784 2.6.  KERMAC_AMD_GRADIENT_L2_MIN_TERMS replaces the rule by a number of terms
// (read on every call, so that a test can send small shapes down the route).
bool gradient_l2_pays(const kmc_norm_gradient_params *p, int64_t tiles_m, int64_t tiles_n)
{
    const char *text = std::getenv("KERMAC_AMD_GRADIENT_L2_MIN_TERMS");
    const double forced = text ? std::atof(text) : 0.0;
    const double terms = static_cast<double>(p->m) * p->n * p->k * p->l;
    if (forced > 0.0) return terms >= forced;
    const int o = p->o;
    const double per_term = o == 1 ? 0.077 : o == 2 ? 0.10 : o == 3 ? 0.126 : o == 4 ? 0.137 : o <= 8 ? 0.028 * o
                          : o <= 16 ? 0.27 : o <= 32 ? 0.56 : 0.0175 * o;
    const double fp32_us = 30.0 + terms * per_term * 1e-6;
    const double padded = static_cast<double>(tiles_m) * tiles_n * kmc::GW_TILE * kmc::GW_TILE * p->k * p->l;
    const double walk_us = padded * 6.3e-9 > 0.056 * p->k ? padded * 6.3e-9 : 0.056 * p->k;
    const double route_us = 200.0 + 1.5e-6 * (static_cast<double>(o) * p->n + p->m) * p->k * p->l + walk_us;
    return (100 + kmc_rules::GRADIENT_L2_ADVANTAGE_PERCENT) * route_us < 100 * fp32_us;
}

bool gradient_l2_layout(const kmc_norm_gradient_params *p, GradientL2Layout *layout)
{
    if (p->norm_type != KMC_NORM_L2 || p->m < 1 || p->n < 1 || p->o < 1 || p->k < 1 || p->l < 1) return false;
    // row r = o * n_rows + n of the product is row n of plane o of e
    if (p->o > 1 && p->e_ld_o != static_cast<int64_t>(p->n) * p->e_ld_n) return false;
    const int64_t rows = static_cast<int64_t>(p->o) * p->n;
    if (rows > 0x7fffffff - kmc::GW_TILE || (p->o + kmc::GL2_OUTPUTS - 1) / kmc::GL2_OUTPUTS > 65535) return false;
    WideLayout &wide = layout->wide;
    wide.tiles_m = (p->m + kmc::GW_TILE - 1) / kmc::GW_TILE;
    wide.tiles_n = static_cast<int>((rows + kmc::GW_TILE - 1) / kmc::GW_TILE);
    if (!gradient_l2_pays(p, wide.tiles_m, wide.tiles_n)) return false;
    if (!place_wide(p->m, static_cast<int>(rows), p->k, p->l, p->a_bs == 0, false, false, &wide)) return false;
    int64_t cursor = wide.bytes;
    layout->products_ld = (p->k + 3) / 4 * 4;
    layout->products = place(cursor, static_cast<int64_t>(p->l) * rows * layout->products_ld * 4);
    layout->shift = place(cursor, static_cast<int64_t>(p->l) * p->n * 4);
    layout->c_transposed = place(cursor, static_cast<int64_t>(p->l) * p->k * p->o * 4);
    layout->g = place(cursor, static_cast<int64_t>(p->l) * p->m * p->o * 4);
    // kmc_matrix_times_coefficients wants a workgroup per CU: 128 columns m and 32 outputs each
    const int64_t workgroups = static_cast<int64_t>((p->m + 127) / 128) * ((p->o + 31) / 32) * p->l;
    int parts = workgroups >= 256 ? 1 : static_cast<int>((256 + workgroups - 1) / workgroups);
    if (parts > p->k / 512) parts = p->k / 512 > 1 ? p->k / 512 : 1;
    if (static_cast<int64_t>(parts) * p->l > 65535) parts = 1;
    layout->g_parts = parts;
    layout->g_partial = parts > 1 ? place(cursor, static_cast<int64_t>(parts) * p->l * p->m * p->o * 4) : 0;
    layout->bytes = cursor;
    return true;
}

}  // namespace

int64_t norm_gradient_l2_wide_bytes(const kmc_norm_gradient_params *p)
{
    GradientL2Layout layout;
    return gradient_l2_layout(p, &layout) ? layout.bytes : 0;
}

// `*taken` says whether the route applied (and the launches were made); if not, nothing was launched.
int launch_norm_gradient_l2_wide(const kmc_norm_gradient_params *p, hipStream_t stream, bool *taken)
{
    *taken = false;
    GradientL2Layout layout;
    if (!p->workspace || !gradient_l2_layout(p, &layout) || p->workspace_bytes < layout.bytes ||
        (reinterpret_cast<uintptr_t>(p->workspace) & (REGION_ALIGN - 1)) != 0)
        return KMC_OK;
    char *workspace = static_cast<char *>(p->workspace);
    const WideLayout &wide = layout.wide;
    const int rows = p->o * p->n;
    const bool scalar_only = (p->flags & KMC_FLAG_FORCE_SCALAR_ACCESS) != 0;

    kmc::GradientL2PrepareArgs prepare = {};
    prepare.b = p->b; prepare.b_ld = p->b_ld; prepare.b_bs = p->b_bs;
    prepare.c = p->c; prepare.c_ld = p->c_ld; prepare.c_bs = p->c_bs;
    prepare.products = reinterpret_cast<float *>(workspace + layout.products);
    prepare.products_ld = layout.products_ld; prepare.products_bs = static_cast<int64_t>(rows) * layout.products_ld;
    prepare.shift = reinterpret_cast<float *>(workspace + layout.shift); prepare.shift_bs = p->n;
    prepare.c_transposed = reinterpret_cast<float *>(workspace + layout.c_transposed);
    prepare.c_transposed_ld = p->o; prepare.c_transposed_bs = static_cast<int64_t>(p->k) * p->o;
    prepare.n = p->n; prepare.o = p->o; prepare.k = p->k;
    hipError_t status = launch(kmc::gradient_l2_products, dim3(p->n, (p->o + kmc::GL2_OUTPUTS - 1) / kmc::GL2_OUTPUTS, p->l),
                               dim3(kmc::GL2_THREADS), stream, prepare);
    if (status != hipSuccess) return fail_hip(status, "gradient_l2_products launch");
    status = launch(kmc::gradient_l2_transpose_c, dim3((p->k + kmc::GL2_THREADS - 1) / kmc::GL2_THREADS, p->l), dim3(kmc::GL2_THREADS), stream, prepare);
    if (status != hipSuccess) return fail_hip(status, "gradient_l2_transpose_c launch");

    // g[m][o] = sum_k a[k][m] c[o][k]: a is a stored panel with m contiguous
    float *g = reinterpret_cast<float *>(workspace + layout.g);
    kmc_matrix_coefficients_params weights = {};
    weights.m = p->m; weights.n = p->k; weights.o = p->o; weights.l = p->l;
    weights.matrix = p->a; weights.matrix_ld = p->a_ld; weights.matrix_bs = p->a_bs;
    weights.coef = prepare.c_transposed; weights.coef_ld = prepare.c_transposed_ld; weights.coef_bs = prepare.c_transposed_bs;
    weights.out = g; weights.out_ld = p->o; weights.out_bs = static_cast<int64_t>(p->m) * p->o;
    if (layout.g_parts > 1) {
        weights.out = reinterpret_cast<float *>(workspace + layout.g_partial);
        weights.n_splits = layout.g_parts;
        weights.out_split_stride = static_cast<int64_t>(p->l) * weights.out_bs;
    }
    const int contracted = kmc_matrix_times_coefficients(&weights, stream);
    if (contracted != KMC_OK) return contracted;
    if (layout.g_parts > 1) {
        kmc::GradientL2SumArgs sum = {};
        sum.partial = weights.out; sum.sum = g;
        sum.count = static_cast<int64_t>(p->l) * weights.out_bs; sum.stride = weights.out_split_stride;
        sum.parts = layout.g_parts;
        status = launch(kmc::gradient_l2_sum_parts, dim3(static_cast<unsigned>((sum.count + kmc::GL2_THREADS - 1) / kmc::GL2_THREADS)),
                        dim3(kmc::GL2_THREADS), stream, sum);
        if (status != hipSuccess) return fail_hip(status, "gradient_l2_sum_parts launch");
    }

    // no centre: the shift of b is in the products already
    kmc::BuildKernelArgs walk = {};
    walk.m = p->m; walk.n = rows; walk.k = p->k; walk.l = p->l;
    const kmc::GramRowsArgs rows_a = rows_args(p->a, p->a_ld, p->a_bs, p->m, KMC_COL_MAJOR, scalar_only, walk, wide, wide.a, workspace);
    const kmc::GramRowsArgs rows_b = rows_args(prepare.products, prepare.products_ld, prepare.products_bs, rows, KMC_ROW_MAJOR, scalar_only,
                                               walk, wide, wide.b, workspace);
    status = launch_gram_rows_pair(rows_a, wide.a.batches, rows_b, wide.b.batches, stream);
    if (status != hipSuccess) return fail_hip(status, "gram_row_stats / gram_f16_split launch");

    kmc::GramWideArgs product = {};
    product.kernel = walk;
    product.kernel.c = p->e; product.kernel.c_ld = p->e_ld_n; product.kernel.c_bs = p->e_bs;
    product.kernel.c_vec = !scalar_only && aligned16(p->e) && p->e_ld_n % 4 == 0 && p->e_bs % 4 == 0;
    product.pieces_a = rows_a.pieces; product.pieces_b = rows_b.pieces;
    product.pieces_a_bs = wide.a.batches > 1 ? wide.a.pieces_bs : 0;
    product.pieces_b_bs = wide.b.batches > 1 ? wide.b.pieces_bs : 0;
    product.squares_a = rows_a.squares; product.squares_b = rows_b.squares;
    product.stats_a_bs = wide.a.batches > 1 ? wide.a.stats_bs : 0;
    product.stats_b_bs = wide.b.batches > 1 ? wide.b.stats_bs : 0;
    product.unscale_a = rows_a.unscale; product.unscale_b = rows_b.unscale;
    product.unscale_a_bs = wide.a.batches > 1 ? wide.a.rows_pad : 0;
    product.unscale_b_bs = wide.b.batches > 1 ? wide.b.rows_pad : 0;
    product.rows_pad_a = wide.a.rows_pad; product.rows_pad_b = wide.b.rows_pad;
    product.slices = wide.slices; product.ranges = wide.ranges;
    product.wide_tiles_m = wide.tiles_m; product.wide_tiles_n = wide.tiles_n; product.wide_tiles_n_padded = wide.tiles_n_padded;
    product.gradient_d = p->d; product.gradient_d_ld = p->d_ld; product.gradient_d_bs = p->d_bs;
    product.gradient_g = g; product.gradient_g_ld = p->o; product.gradient_g_bs = weights.out_bs;
    product.gradient_shift = prepare.shift; product.gradient_shift_bs = prepare.shift_bs;
    product.gradient_n = p->n;
    const dim3 grid(static_cast<unsigned>(wide.tiles_m) * wide.tiles_n_padded, p->l, 1);
    status = launch(kmc::gram_f16_wide<false, kmc::GW_EPILOGUE_GRADIENT_L2>, grid, dim3(kmc::GW_THREADS), stream, product);
    if (status != hipSuccess) return fail_hip(status, "gram_f16_wide (gradient) launch");
    *taken = true;
    return KMC_OK;
}

}  // namespace kmc_host
