// Copies of the operands as padded k-major panels, for the direct kernel's variant with b in scalar registers.
//
// build_kernel_scalar_b (build_kernel_scalar_b.hpp) is the fastest direct kernel for absolute and squared
// differences of large problems, but it takes its operands one way only: rows contiguous (x[k][row]), 16-byte
// aligned, K a multiple of 16 and, for b, rows of a multiple of 16 columns.  Operands as torch allocates them
// (k contiguous), misaligned views, and shapes with other K or N run the three-wave kernel, 5 to 7 % slower.  With
// KMC_FLAG_DIRECT_PANELS and a workspace, kmc_build_kernel copies the operands that do not fit into panels that
// do -- [entry][k rounded up to 16][rows rounded up to 64], zeros in the padding (a zero in both operands adds
// |0 - 0| = 0 to a sum, and padded columns of b are computed but not stored; a panel against itself is copied once)
// -- and launches that kernel on the copies.  A copy reads and writes its operand once: 0.1 ms for 30000 x 1024 against the 1.5 ms the kernel gains
// at M = N = 30000.  The sums are those of the direct kernels bit for bit (same terms, same order).
// The reference has one kernel for all storage orders (include/build_a_kernel.cuh:484-539) and no copies.
#include <hip/hip_runtime.h>

#include "../host/host_common.hpp"
#include "../host/dispatch_rules.hpp"
#include "build_kernel_scalar_b.hpp"
#include "launch.hpp"

namespace kmc {

constexpr int PC_TILE = 64;          // rows x k per workgroup
constexpr int PC_THREADS = 256;
constexpr int PC_ROW_PAD = 64;       // rows of a panel are padded to a multiple of this

struct PanelCopyArgs {
    const float *source; i64 ld, bs;  // [row][k] with k contiguous (k_contiguous) or [k][row]
    int k_contiguous;
    int rows, k;                      // what exists in the source
    float *panel;                     // [entry][k_padded][rows_padded]
    int rows_padded, k_padded;
};

// grid: (rows_padded / 64, k_padded / 64 rounded up, entries).  Reads run along the contiguous index of the source,
// writes along the rows of the panel; the tile turns in LDS (pitch 65: no bank is hit twice either way).
__global__ __launch_bounds__(PC_THREADS) void panel_copy(const PanelCopyArgs args)
{
    __shared__ float tile[PC_TILE][PC_TILE + 1];      // [row][k]
    const int t = threadIdx.x;
    const int along = t & 63, across = t >> 6;
    const int row0 = blockIdx.x * PC_TILE, k0 = blockIdx.y * PC_TILE;
    const float *source = args.source + (i64)blockIdx.z * args.bs;
    if (args.k_contiguous) {
        const int k = k0 + along;
#pragma unroll 4
        for (int i = across; i < PC_TILE; i += PC_THREADS / 64) {
            const int row = row0 + i;
            tile[i][along] = row < args.rows && k < args.k ? source[(i64)row * args.ld + k] : 0.0f;
        }
    } else {
        const int row = row0 + along;
#pragma unroll 4
        for (int i = across; i < PC_TILE; i += PC_THREADS / 64) {
            const int k = k0 + i;
            tile[along][i] = row < args.rows && k < args.k ? source[(i64)k * args.ld + row] : 0.0f;
        }
    }
    __syncthreads();
    float *panel = args.panel + (i64)blockIdx.z * args.k_padded * args.rows_padded;
#pragma unroll 4
    for (int i = across; i < PC_TILE; i += PC_THREADS / 64) {
        const int k = k0 + i;
        if (k < args.k_padded) panel[(i64)k * args.rows_padded + row0 + along] = tile[along][i];
    }
}

}  // namespace kmc

namespace kmc_host {

namespace {

struct PanelPlan {
    bool copy_a, copy_b;
    int k_padded, m_padded, n_padded;
    int entries_a, entries_b;          // 1 for an operand that every batch entry shares
    int64_t bytes_a, bytes_b;          // multiples of 256
};

int64_t round_up(int64_t x, int64_t to) { return (x + to - 1) / to * to; }

// Whether kmc_build_kernel, given KMC_FLAG_DIRECT_PANELS and room, runs this call on copies, and which.
bool plan_panels(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, PanelPlan *plan)
{
    if (!(p->flags & KMC_FLAG_DIRECT_PANELS)) return false;
    if (p->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16 | KMC_FLAG_DOT_PIECES | KMC_FLAG_L1_FIXED | KMC_FLAG_FORCE_SCALAR_ACCESS)) return false;
    // the inner powers build_kernel_scalar_b exists for: |x|, x^2, and the scalar exponents 3 and 4 that kmc_build_kernel evaluates as products
    const bool cube_or_fourth = p->inner_power == KMC_POW_POW && !p->p_inner && !(p->flags & KMC_FLAG_GENERIC_POWER) &&
                                (p->p_inner_value == 3.0f || p->p_inner_value == 4.0f);
    if (p->inner_operator != KMC_OP_DIFF || (p->inner_power != KMC_POW_ABS && p->inner_power != KMC_POW_SQUARE && !cube_or_fourth)) return false;
    if (args.k_total != 0 || args.repair_only || args.m < 1 || args.n < 1 || args.k < 1 || args.l < 1) return false;
    if (!args.c_vec) return false;
    const int64_t tiles_m = ceil_div(args.m, kmc::SB_TILE_M), tiles_n = ceil_div(args.n, kmc::SB_TILE_N);
    // a panel against itself: the kernel runs the tiles that reach the diagonal or lie below it, and has a size rule of its own for them
    const int64_t tiles = args.symmetric ? 2 * (tiles_m - 1) * tiles_m + (4 * tiles_m < tiles_n ? 4 * tiles_m : tiles_n) : tiles_m * tiles_n;
    const int64_t enough = args.symmetric ? kmc_rules::DIRECT_SCALAR_B_MIN_TILES_SYMMETRIC : kmc_rules::DIRECT_PANELS_MIN_TILES;
    const bool any_size = p->flags & KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE;
    if (!any_size && (tiles < enough || args.k < kmc_rules::DIRECT_PANELS_MIN_K)) return false;
    if (tiles > 0x7fffffff) return false;
    auto fits = [&](const float *x, int64_t ld, int64_t bs, int majorness) {
        return majorness == KMC_COL_MAJOR && aligned16(x) && ld % 4 == 0 && bs % 4 == 0;
    };
    const bool k_fits = args.k % kmc::BK_TILE_K == 0;
    plan->copy_a = !k_fits || !fits(p->a, p->a_ld, p->a_bs, p->a_majorness);
    plan->copy_b = !k_fits || !fits(p->b, p->b_ld, p->b_bs, p->b_majorness) || args.n % kmc::SB_WAVE_N != 0;
    if (!plan->copy_a && !plan->copy_b) return false;       // the ordinary launch takes the kernel by itself
    plan->k_padded = static_cast<int>(round_up(args.k, kmc::BK_TILE_K));
    plan->m_padded = static_cast<int>(round_up(args.m, kmc::PC_ROW_PAD));
    plan->n_padded = static_cast<int>(round_up(args.n, kmc::PC_ROW_PAD));
    plan->entries_a = p->a_bs == 0 ? 1 : args.l;
    plan->entries_b = p->b_bs == 0 ? 1 : args.l;
    plan->bytes_a = plan->copy_a ? round_up(4ll * plan->entries_a * plan->k_padded * plan->m_padded, 256) : 0;
    plan->bytes_b = plan->copy_b ? round_up(4ll * plan->entries_b * plan->k_padded * plan->n_padded, 256) : 0;
    if (args.symmetric) {
        // one panel on both sides: one copy
        plan->copy_a = plan->copy_b = true;
        plan->bytes_a = round_up(4ll * plan->entries_a * plan->k_padded * plan->m_padded, 256);
        plan->bytes_b = 0;
    }
    return true;
}

hipError_t copy_panel(const float *source, int64_t ld, int64_t bs, int majorness, int rows, int k, int entries, float *panel,
                      int rows_padded, int k_padded, hipStream_t stream)
{
    kmc::PanelCopyArgs copy;
    copy.source = source; copy.ld = ld; copy.bs = bs;
    copy.k_contiguous = majorness == KMC_COL_MAJOR ? 0 : 1;
    copy.rows = rows; copy.k = k;
    copy.panel = panel; copy.rows_padded = rows_padded; copy.k_padded = k_padded;
    const dim3 grid(rows_padded / kmc::PC_TILE, static_cast<unsigned>(ceil_div(k_padded, kmc::PC_TILE)), entries);
    return launch(kmc::panel_copy, grid, dim3(kmc::PC_THREADS), stream, copy);
}

}  // namespace

// Bytes of workspace kmc_build_kernel wants for copies of the operands of this call; 0: none are made.
int64_t direct_panels_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args)
{
    PanelPlan plan;
    if (!plan_panels(p, args, &plan)) return 0;
    if (plan.k_padded / kmc::PC_TILE + 1 > 65535 || args.l > 65535) return 0;
    return plan.bytes_a + plan.bytes_b;
}

// Copies what has to be copied into the workspace of `p` and points `args` at the copies (operands, strides, k
// rounded up when both are copies, panels); *taken says whether it did.  The caller then launches the direct
// kernel with both loaders LOAD_COL_VEC, which picks build_kernel_scalar_b by its own rule.
hipError_t launch_direct_panels(const kmc_build_kernel_params *p, kmc::BuildKernelArgs *args, hipStream_t stream, bool *taken)
{
    *taken = false;
    PanelPlan plan;
    const int64_t needed = direct_panels_bytes(p, *args);
    if (needed == 0 || !plan_panels(p, *args, &plan)) return hipSuccess;
    if (!p->gram_workspace || p->gram_workspace_bytes < needed || (reinterpret_cast<uintptr_t>(p->gram_workspace) & 255) != 0)
        return hipSuccess;
    char *workspace = static_cast<char *>(p->gram_workspace);
    if (plan.copy_a) {
        float *panel = reinterpret_cast<float *>(workspace);
        hipError_t e = copy_panel(p->a, p->a_ld, p->a_bs, p->a_majorness, args->m, args->k, plan.entries_a, panel, plan.m_padded,
                                  plan.k_padded, stream);
        if (e != hipSuccess) return e;
        args->a = panel;
        args->a_ld = plan.m_padded;
        args->a_bs = plan.entries_a == 1 ? 0 : static_cast<int64_t>(plan.k_padded) * plan.m_padded;
    }
    if (args->symmetric) {
        args->b = args->a; args->b_ld = args->a_ld; args->b_bs = args->a_bs;
        args->panels |= kmc::BK_PANELS_B_PADDED;
    } else if (plan.copy_b) {
        float *panel = reinterpret_cast<float *>(workspace + plan.bytes_a);
        hipError_t e = copy_panel(p->b, p->b_ld, p->b_bs, p->b_majorness, args->n, args->k, plan.entries_b, panel, plan.n_padded,
                                  plan.k_padded, stream);
        if (e != hipSuccess) return e;
        args->b = panel;
        args->b_ld = plan.n_padded;
        args->b_bs = plan.entries_b == 1 ? 0 : static_cast<int64_t>(plan.k_padded) * plan.n_padded;
        args->panels |= kmc::BK_PANELS_B_PADDED;
    }
    args->k = plan.k_padded;        // a multiple of 16 already, or both operands are copies with zeros past k
    args->panels |= kmc::BK_PANELS_COPIED;
    *taken = true;
    return hipSuccess;
}

}  // namespace kmc_host
