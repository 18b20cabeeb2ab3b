// Host side of the fixed-point path for sums of absolute differences (l1_fixed.hpp): when it
// applies, how the caller's workspace is divided, and the launches.
#include <hip/hip_runtime.h>

#include "../host/host_common.hpp"
#include "../host/dispatch_rules.hpp"
#include "launch.hpp"
#include "l1_fixed.hpp"

namespace kmc_host {

namespace {

constexpr int64_t REGION_ALIGN = 256;
constexpr int SAMPLE_TILES = 1024;      // over the batch, 256 pairs each; at least 64 per batch entry

// Whether the route pays: it adds seven small launches and two passes over the operands (about
// 16 bytes per operand element) to a walk that takes 0.85 of the direct kernel's time, so it needs
// a problem whose walk is long against both.  (KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE sets the rule aside.)
bool fixed_pays(int64_t tiles, int k)
{
    return tiles >= kmc_rules::L1_FIXED_MIN_TILES && k >= kmc_rules::L1_FIXED_MIN_K;
}

struct FixedLayout {
    int k_padded, m_padded, n_padded, bits;
    bool same_panel;
    int64_t header, qa, qb;      // byte offsets into the workspace
    int64_t qa_bs, qb_bs;        // words per batch entry
    int64_t bytes;
};

int64_t place(int64_t &cursor, int64_t bytes)
{
    const int64_t at = cursor;
    cursor = (cursor + bytes + REGION_ALIGN - 1) / REGION_ALIGN * REGION_ALIGN;
    return at;
}

bool fixed_layout(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, FixedLayout *layout)
{
    if (!(p->flags & KMC_FLAG_L1_FIXED) || p->inner_operator != KMC_OP_DIFF || p->inner_power != KMC_POW_ABS) return false;
    if (args.m < 1 || args.n < 1 || args.l < 1 || args.k < 1 || args.k_total != 0) return false;
    const int64_t tiles_m = args.tiles_m;
    const int64_t tiles = args.symmetric ? tiles_m * (tiles_m + 1) / 2 : tiles_m * args.tiles_n;
    if (!(p->flags & KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE) && !fixed_pays(tiles * args.l, args.k)) return false;
    layout->k_padded = (args.k + kmc::BK_TILE_K - 1) / kmc::BK_TILE_K * kmc::BK_TILE_K;
    layout->m_padded = args.tiles_m * kmc::BK_TILE_M;
    layout->n_padded = args.tiles_n * kmc::BK_TILE_N;
    layout->bits = args.k <= 64 ? 26 : args.k <= 256 ? 24 : 22;      // l1_fixed_bits
    layout->same_panel = p->a == p->b && p->m == p->n && p->a_ld == p->b_ld && p->a_bs == p->b_bs &&
                         p->a_majorness == p->b_majorness;
    int64_t cursor = 0;
    layout->header = place(cursor, static_cast<int64_t>(args.l) * sizeof(kmc::L1FixedHeader));
    // every batch entry has a grid of its own, so an operand that is the same for all of them is
    // converted for each
    layout->qa_bs = static_cast<int64_t>(layout->k_padded) * layout->m_padded;
    layout->qa = place(cursor, args.l * layout->qa_bs * 4);
    if (layout->same_panel) {
        layout->qb_bs = layout->qa_bs;
        layout->qb = layout->qa;
    } else {
        layout->qb_bs = static_cast<int64_t>(layout->k_padded) * layout->n_padded;
        layout->qb = place(cursor, args.l * layout->qb_bs * 4);
    }
    layout->bytes = cursor;
    return true;
}

kmc::L1FixedPanel panel_of(const float *x, int64_t ld, int64_t bs, int majorness, int rows, int rows_padded, char *workspace,
                           int64_t offset, int64_t q_bs)
{
    kmc::L1FixedPanel panel;
    panel.x = x; panel.ld = ld; panel.bs = bs;
    panel.majorness = majorness == KMC_COL_MAJOR ? 0 : 1;
    panel.rows = rows;
    panel.q = reinterpret_cast<unsigned *>(workspace + offset);
    panel.q_ld = rows_padded;
    panel.q_bs = q_bs;
    return panel;
}

}  // namespace

int64_t l1_fixed_bytes(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args)
{
    FixedLayout layout;
    return fixed_layout(p, args, &layout) ? layout.bytes : 0;
}

void forget_split_in(const void *workspace);      // gram_f16_wide_inst.hip

// *taken = the walk was launched: the caller follows it with the direct kernel in repair mode.
hipError_t launch_l1_fixed(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, hipStream_t stream, bool *taken)
{
    *taken = false;
    FixedLayout layout;
    if (!p->gram_workspace || (reinterpret_cast<uintptr_t>(p->gram_workspace) & (REGION_ALIGN - 1)) != 0) return hipSuccess;
    if (!fixed_layout(p, args, &layout) || p->gram_workspace_bytes < layout.bytes) return hipSuccess;
    if (args.l > 65535 || layout.k_padded / 64 + 1 > 65535) return hipSuccess;
    char *workspace = static_cast<char *>(p->gram_workspace);
    forget_split_in(workspace);

    kmc::L1FixedArgs fixed;
    fixed.kernel = args;
    fixed.a = panel_of(p->a, p->a_ld, p->a_bs, p->a_majorness, args.m, layout.m_padded, workspace, layout.qa, layout.qa_bs);
    fixed.b = panel_of(p->b, p->b_ld, p->b_bs, p->b_majorness, args.n, layout.n_padded, workspace, layout.qb, layout.qb_bs);
    fixed.header = reinterpret_cast<kmc::L1FixedHeader *>(workspace + layout.header);
    fixed.bits = layout.bits;
    fixed.k_padded = layout.k_padded;
    fixed.tolerance = p->gram_trust > 0.0f && p->gram_trust < 1.0f ? p->gram_trust : 8e-6f;
    fixed.sample_tiles = SAMPLE_TILES / args.l > 64 ? SAMPLE_TILES / args.l : 64;

    void *clear_args[] = {&fixed.header, const_cast<int *>(&args.l)};
    hipError_t e = hipLaunchKernel(reinterpret_cast<const void *>(kmc::l1_fixed_clear), dim3((args.l * 16 + kmc::L1F_THREADS - 1) / kmc::L1F_THREADS),
                                   dim3(kmc::L1F_THREADS), clear_args, 0, stream);
    if (e != hipSuccess) return e;
    int k = args.k;
    for (int side = 0; side < (layout.same_panel ? 1 : 2); side++) {
        kmc::L1FixedPanel &panel = side == 0 ? fixed.a : fixed.b;
        const int lines = panel.majorness == 0 ? k : panel.rows;
        void *range_args[] = {&panel, &k, &fixed.header};
        e = hipLaunchKernel(reinterpret_cast<const void *>(kmc::l1_fixed_range), dim3(lines < 2048 ? lines : 2048, args.l),
                            dim3(kmc::L1F_THREADS), range_args, 0, stream);
        if (e != hipSuccess) return e;
    }
    e = launch(kmc::l1_fixed_sample, dim3(fixed.sample_tiles, args.l), dim3(kmc::L1F_THREADS), stream, fixed);
    if (e != hipSuccess) return e;
    for (int side = 0; side < (layout.same_panel ? 1 : 2); side++) {
        kmc::L1FixedPanel &panel = side == 0 ? fixed.a : fixed.b;
        void *convert_args[] = {&panel, &k, &fixed.k_padded, &fixed.bits, &fixed.header};
        e = hipLaunchKernel(reinterpret_cast<const void *>(kmc::l1_fixed_convert),
                            dim3(static_cast<unsigned>(panel.q_ld / 64), (layout.k_padded + 63) / 64, args.l), dim3(kmc::L1F_THREADS),
                            convert_args, 0, stream);
        if (e != hipSuccess) return e;
    }
    e = launch(kmc::l1_fixed_kernel, dim3(static_cast<unsigned>(args.grid_width), args.l), dim3(kmc::BK_THREADS), stream, fixed);
    if (e != hipSuccess) return e;
    *taken = true;
    return hipSuccess;
}

}  // namespace kmc_host
