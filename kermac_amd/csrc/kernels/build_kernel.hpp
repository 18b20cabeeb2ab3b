// Fused pairwise-reduction kernel for gfx950:
//
//   C[m, n, l] = kernel_fn( outer( sum_k inner( B[n,k,l] (- or *) A[m,k,l] ) ) )
//
// Replaces the reference's cute_build_kernel (include/build_a_kernel.cuh:541-623)
// with a design written for CDNA4 wave64 hardware:
//
//   * one workgroup of 256 lanes (4 waves) owns a 128 x 128 output tile and walks
//     K in slices of 16;
//   * each lane owns an 8 x 8 register tile made of 4-wide contiguous pieces, so
//     every LDS fragment read is one ds_read_b128 and every output store is one
//     128-bit store along the contiguous M direction;
//   * HBM -> register -> LDS staging is double buffered: the loads for slice
//     t+1 are in flight while slice t is consumed, with one barrier per slice;
//   * the inner loop is nothing but subtract + accumulate on the fp32 VALU
//     (|x| and negation ride on source modifiers), 2 issue slots per (m,n,k);
//   * outer power, epsilon mask, Laplace/Gaussian function and the diagonal
//     regularisation are applied to the registers right before the store.
//
// Output is always written "column major": C[m + n * c_ld + l * c_bs].  The host
// swaps the operands when the caller's out tensor is row major, exactly as the
// reference does (src/kermac/build_a_kernel.py:323-336).
#pragma once

#include "device_common.hpp"

namespace kmc {

struct BuildKernelArgs {
    int m, n, k, l;
    const float *a; i64 a_ld, a_bs;  // A: m x k panel
    const float *b; i64 b_ld, b_bs;  // B: n x k panel
    float *c; i64 c_ld, c_bs;        // C: m x n, m contiguous
    // Hyper-parameters: a device pointer indexed [l * stride], or (pointer null) the value.
    const float *p_inner; i64 p_inner_bs;
    const float *p_outer; i64 p_outer_bs;
    const float *bandwidth; i64 bandwidth_bs;
    const float *regularization; i64 regularization_bs;
    float p_inner_value, p_outer_value, bandwidth_value, regularization_value;
    int reg_off_x, reg_off_y;
    float epsilon;
    float diff_sign;   // +1, or -1 when the host swapped the operands
    int outer_power, kernel_type;
    int c_vec;     // c, c_ld and c_bs are multiples of 16 bytes: 128-bit stores allowed
    int tiles_m, tiles_n;
    int tiles_n_padded;  // tiles_n, rounded up to a multiple of 8 where that adds little; grid.x = tiles_m * tiles_n_padded
    int repair_only;     // recompute only the tiles that carry BK_REPAIR_MARKER (see gram_kernel.hpp)
    int symmetric;       // A and B are the same panel and the result is symmetric: only tiles with
                         // tile_m >= tile_n are computed, each is also stored mirrored
    float gram_trust;    // gram_kernel.hpp: distrust d^2 below gram_trust * (|a|^2 + |b|^2)
    int k_total;         // 0, or: the batch entries are consecutive ranges of k terms of one contraction of
                         // k_total terms, and the last entry walks only what is left
    int grid_width;      // gridDim.x: tiles_m * tiles_n_padded, or (symmetric) the tiles of one triangle
    // Matrix-core kernels only: a point c[k] (per batch entry, padded with zeros to a multiple of
    // GRAM_CENTRE_PAD floats, 16-byte aligned) that is subtracted from both operands while they are
    // staged; null: nothing is subtracted.
    const float *centre; i64 centre_bs;
    // Matrix-core kernels for squared differences only, or null: what a sample of the result said before the
    // launch (gram_probe.hip fills it, sample_leaves_it_to_the_direct_kernel reads it).
    const unsigned *sample;
    // build_kernel_scalar_b only.  BK_PANELS_COPIED: the operands are the copies of panel_copy.hip, made for that
    // kernel, which therefore runs whatever the size of the problem.  BK_PANELS_B_PADDED: the rows of b hold n rounded
    // up to 16 columns (zeros past n), so that a wave's 16 columns can always be loaded; columns below n are stored.
    int panels;
};

constexpr int BK_PANELS_COPIED = 1;
constexpr int BK_PANELS_B_PADDED = 2;

constexpr int GRAM_CENTRE_PAD = 64;

// The sample taken in front of a matrix-core launch for squared differences: BK_SAMPLE_TILES tiles of 128 x 128
// of the result, 16 rows of each operand from each, their 256 pairs.  One word per sampled tile: pairs below
// the trust threshold in the low half, 1 in the high half when there are any.
constexpr int BK_SAMPLE_TILES = 256;
constexpr int BK_SAMPLE_ROWS = 16;
constexpr int BK_SAMPLE_BYTES = BK_SAMPLE_TILES * 4;
constexpr int BK_SAMPLE_LEAVE_PER_16384 = 2;     // pairs below the threshold, spread over the tiles: leave the call to the direct kernel

// What the sample says: true when the matrix cores' work would be thrown away.  A 128 x 128 part with one pair
// below the trust threshold is recomputed whole by the repair launch, so pairs below the threshold cost the
// matrix cores' work when they sit in (nearly) every part: 2 such pairs in 16384, spread evenly, already put one
// into six parts of seven.  The same share of pairs packed into few parts -- points stored cluster by cluster,
// whose near-duplicates fill the blocks on the diagonal -- costs the repair of those parts only.  The two are
// told apart by the number of sampled tiles that show such a pair: spread evenly over the sampled tiles, `below`
// pairs land in tiles (1 - exp(-below / tiles)) different ones; packed, in far fewer.
// Every lane of a wave calls it; the answer is the same for every wave of the launch.
__device__ __forceinline__ bool sample_leaves_it_to_the_direct_kernel(const unsigned *sample)
{
    static_assert(BK_SAMPLE_TILES == 256, "a lane reads four words");
    const uint4 words = reinterpret_cast<const uint4 *>(sample)[threadIdx.x & 63];
    unsigned below = (words.x & 0xffffu) + (words.y & 0xffffu) + (words.z & 0xffffu) + (words.w & 0xffffu);
    unsigned tiles_below = (words.x >> 16) + (words.y >> 16) + (words.z >> 16) + (words.w >> 16);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        below += (unsigned)__shfl_xor((int)below, offset);
        tiles_below += (unsigned)__shfl_xor((int)tiles_below, offset);
    }
    const float pairs = (float)(BK_SAMPLE_TILES * BK_SAMPLE_ROWS * BK_SAMPLE_ROWS);
    if ((float)below * 16384.0f < (float)BK_SAMPLE_LEAVE_PER_16384 * pairs) return false;
    const float spread = (float)BK_SAMPLE_TILES * (1.0f - __expf(-(float)below / (float)BK_SAMPLE_TILES));
    return (float)tiles_below >= 0.7f * spread;
}

constexpr int BK_TILE_M = 128;
constexpr int BK_TILE_N = 128;
constexpr int BK_TILE_K = 16;
constexpr int BK_THREADS = 256;
constexpr int BK_XCDS = 8;     // MI355X: 8 accelerator dies, 32 CUs and one L2 each
#ifndef BK_BAND_TILES
#define BK_BAND_TILES 64
#endif
constexpr int BK_BAND_N = BK_BAND_TILES;  // height, in tiles, of the bands the tile order walks: 8 per XCD
// Row pitch of an LDS slice in floats.  +4 keeps rows 16-byte aligned and skews
// the banks so that the transposing (k-contiguous) loaders write conflict-free.
constexpr int BK_LDS_PITCH = BK_TILE_M + 4;
constexpr int BK_LDS_SLICE = BK_TILE_K * BK_LDS_PITCH;

// One operand's share of a 128 x 16 slice: 8 floats per lane.  `row` is the m (or
// n) index inside the tile, `kk` the k index inside the slice.
template <int MODE>
struct TileLoader {
    const float *ptr;   // this lane's first element of the current slice
    i64 step;           // pointer advance per slice
    i64 ld;
    int lane_row, lane_k;

    __device__ __forceinline__ void init(const float *base, i64 ld_, int row0, int tid)
    {
        ld = ld_;
        if (MODE == LOAD_COL_VEC) {
            lane_row = (tid & 31) * 4; lane_k = tid >> 5;          // rows +0..3, k +0 / +8
            ptr = base + (i64)lane_k * ld + row0 + lane_row; step = (i64)BK_TILE_K * ld;
        } else if (MODE == LOAD_COL_SCALAR) {
            lane_row = tid & 127; lane_k = tid >> 7;               // k + 2 i
            ptr = base + (i64)lane_k * ld + row0 + lane_row; step = (i64)BK_TILE_K * ld;
        } else if (MODE == LOAD_ROW_VEC) {
            lane_row = tid >> 2; lane_k = (tid & 3) * 4;           // rows +0 / +64, k +0..3
            ptr = base + (i64)(row0 + lane_row) * ld + lane_k; step = BK_TILE_K;
        } else {
            lane_row = tid >> 4; lane_k = tid & 15;                // rows + 16 i
            ptr = base + (i64)(row0 + lane_row) * ld + lane_k; step = BK_TILE_K;
        }
    }

    // (row, k) of register i inside the tile / slice, and its offset from ptr.
    __device__ __forceinline__ int row_of(int i) const
    {
        if (MODE == LOAD_COL_VEC) return lane_row + (i & 3);
        if (MODE == LOAD_COL_SCALAR) return lane_row;
        if (MODE == LOAD_ROW_VEC) return lane_row + (i >> 2) * 64;
        return lane_row + 16 * i;
    }
    __device__ __forceinline__ int k_of(int i) const
    {
        if (MODE == LOAD_COL_VEC) return lane_k + (i >> 2) * 8;
        if (MODE == LOAD_COL_SCALAR) return lane_k + 2 * i;
        if (MODE == LOAD_ROW_VEC) return lane_k + (i & 3);
        return lane_k;
    }
    __device__ __forceinline__ i64 offset_of(int i) const
    {
        if (MODE == LOAD_COL_VEC) return (i64)(i >> 2) * 8 * ld + (i & 3);
        if (MODE == LOAD_COL_SCALAR) return (i64)(2 * i) * ld;
        if (MODE == LOAD_ROW_VEC) return (i64)(i >> 2) * 64 * ld + (i & 3);
        return (i64)(16 * i) * ld;
    }

    // Row of register i relative to lane_row (a compile-time constant per mode), how
    // many lanes hold registers of the same row, and this lane's index among them.
    // Used by kernels that reduce per-row quantities over what the lanes staged.
    static __device__ __forceinline__ constexpr int row_offset_of(int i)
    {
        return MODE == LOAD_COL_VEC ? (i & 3) : MODE == LOAD_COL_SCALAR ? 0 : MODE == LOAD_ROW_VEC ? (i >> 2) * 64 : 16 * i;
    }
    static __device__ __forceinline__ constexpr int lanes_per_row()
    {
        return MODE == LOAD_COL_VEC ? 8 : MODE == LOAD_COL_SCALAR ? 2 : MODE == LOAD_ROW_VEC ? 4 : 16;
    }
    static __device__ __forceinline__ int share_index(int tid)
    {
        return MODE == LOAD_COL_VEC ? tid >> 5 : MODE == LOAD_COL_SCALAR ? tid >> 7 : MODE == LOAD_ROW_VEC ? tid & 3 : tid & 15;
    }

    // Whole slice inside the matrix: no predicates.
    __device__ __forceinline__ void load_full(float (&r)[8]) const
    {
        if (MODE == LOAD_COL_VEC || MODE == LOAD_ROW_VEC) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const float4 v = *reinterpret_cast<const float4 *>(ptr + offset_of(4 * h));
                r[4 * h + 0] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = ptr[offset_of(i)];
        }
    }

    // Edge slice: rows >= rows_valid or k >= k_valid read as 0.  A zero in both
    // operands contributes inner(0) = 0 for every inner power the kernel offers
    // (the reference zero-fills its shared-memory tiles the same way,
    // include/build_a_kernel.cuh:203-252).
    __device__ __forceinline__ void load_edge(float (&r)[8], int rows_valid, int k_valid) const
    {
        if (MODE == LOAD_COL_VEC || MODE == LOAD_ROW_VEC) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const bool all_in = row_of(4 * h + 3) < rows_valid && k_of(4 * h + 3) < k_valid;
                if (all_in) {
                    const float4 v = *reinterpret_cast<const float4 *>(ptr + offset_of(4 * h));
                    r[4 * h + 0] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int i = 4 * h + j;
                        r[i] = (row_of(i) < rows_valid && k_of(i) < k_valid) ? ptr[offset_of(i)] : 0.0f;
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                r[i] = (row_of(i) < rows_valid && k_of(i) < k_valid) ? ptr[offset_of(i)] : 0.0f;
            }
        }
    }

    __device__ __forceinline__ void advance() { ptr += step; }

    // c[i] = centre[k of register i] for the current slice; `slice_centre` points at the slice's
    // first k.  No predicates: the vector is padded with zeros past K.
    __device__ __forceinline__ void load_centre(float (&c)[8], const float *slice_centre) const
    {
        if (MODE == LOAD_COL_VEC) {
            const float lo = slice_centre[lane_k], hi = slice_centre[lane_k + 8];
#pragma unroll
            for (int i = 0; i < 8; i++) c[i] = i < 4 ? lo : hi;
        } else if (MODE == LOAD_COL_SCALAR) {
#pragma unroll
            for (int i = 0; i < 8; i++) c[i] = slice_centre[lane_k + 2 * i];
        } else if (MODE == LOAD_ROW_VEC) {
            const float4 v = *reinterpret_cast<const float4 *>(slice_centre + lane_k);
            c[0] = c[4] = v.x; c[1] = c[5] = v.y; c[2] = c[6] = v.z; c[3] = c[7] = v.w;
        } else {
            const float v = slice_centre[lane_k];
#pragma unroll
            for (int i = 0; i < 8; i++) c[i] = v;
        }
    }

    // Write the 8 registers into one LDS slice laid out [k][row] with pitch BK_LDS_PITCH.
    __device__ __forceinline__ void store(float *slice, const float (&r)[8]) const
    {
        if (MODE == LOAD_COL_VEC) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                *reinterpret_cast<float4 *>(slice + (lane_k + 8 * h) * BK_LDS_PITCH + lane_row) =
                    make_float4(r[4 * h], r[4 * h + 1], r[4 * h + 2], r[4 * h + 3]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) slice[k_of(i) * BK_LDS_PITCH + row_of(i)] = r[i];
        }
    }
};

// One row of the register tile for the two transcendental-free distance kernels,
// written out as 8 independent subtractions followed by 8 independent
// accumulations, so that no instruction waits on the one issued just before it
// (the compiler's own schedule pairs each subtraction with its dependent
// accumulate; measured on the same board that costs 1 % for |x| and 5 % for x^2).
#define KMC_SUB8 \
    "v_sub_f32 %8, %24, %16\n\tv_sub_f32 %9, %24, %17\n\tv_sub_f32 %10, %24, %18\n\tv_sub_f32 %11, %24, %19\n\t" \
    "v_sub_f32 %12, %24, %20\n\tv_sub_f32 %13, %24, %21\n\tv_sub_f32 %14, %24, %22\n\tv_sub_f32 %15, %24, %23\n\t"
#define KMC_ROW_OPERANDS(accrow, fa, b) \
    : "+v"(accrow[0]), "+v"(accrow[1]), "+v"(accrow[2]), "+v"(accrow[3]), "+v"(accrow[4]), "+v"(accrow[5]), \
      "+v"(accrow[6]), "+v"(accrow[7]), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), \
      "=&v"(t6), "=&v"(t7) \
    : "v"(fa[0]), "v"(fa[1]), "v"(fa[2]), "v"(fa[3]), "v"(fa[4]), "v"(fa[5]), "v"(fa[6]), "v"(fa[7]), "v"(b)

__device__ __forceinline__ void row_abs_diff(float (&accrow)[8], const float (&fa)[8], float b)
{
    float t0, t1, t2, t3, t4, t5, t6, t7;
    asm volatile(KMC_SUB8
                 "v_add_f32 %0, |%8|, %0\n\tv_add_f32 %1, |%9|, %1\n\tv_add_f32 %2, |%10|, %2\n\t"
                 "v_add_f32 %3, |%11|, %3\n\tv_add_f32 %4, |%12|, %4\n\tv_add_f32 %5, |%13|, %5\n\t"
                 "v_add_f32 %6, |%14|, %6\n\tv_add_f32 %7, |%15|, %7"
                 KMC_ROW_OPERANDS(accrow, fa, b));
}

__device__ __forceinline__ void row_square_diff(float (&accrow)[8], const float (&fa)[8], float b)
{
    float t0, t1, t2, t3, t4, t5, t6, t7;
    asm volatile(KMC_SUB8
                 "v_fmac_f32 %0, %8, %8\n\tv_fmac_f32 %1, %9, %9\n\tv_fmac_f32 %2, %10, %10\n\t"
                 "v_fmac_f32 %3, %11, %11\n\tv_fmac_f32 %4, %12, %12\n\tv_fmac_f32 %5, %13, %13\n\t"
                 "v_fmac_f32 %6, %14, %14\n\tv_fmac_f32 %7, %15, %15"
                 KMC_ROW_OPERANDS(accrow, fa, b));
}

// |b - a|^p as exp2(p * log2|b - a|) for one row: 8 subtractions, 8 v_log_f32, 8
// multiplications, 8 v_exp_f32, 8 accumulations.  The compiler's own schedule
// runs each element's five dependent instructions back to back through one or
// two temporaries; grouped, every instruction has seven independent ones between
// itself and its producer (which also covers the wait state a vector instruction
// needs before it may read the result of a transcendental one).  The loop is
// bound by the issue rate of the two transcendentals either way: measured on the
// same board the grouping is worth 0.6 %.
__device__ __forceinline__ void row_pow_diff(float (&accrow)[8], const float (&fa)[8], float b, float p)
{
    float t0, t1, t2, t3, t4, t5, t6, t7;
    asm volatile(KMC_SUB8
                 "v_log_f32 %8, |%8|\n\tv_log_f32 %9, |%9|\n\tv_log_f32 %10, |%10|\n\tv_log_f32 %11, |%11|\n\t"
                 "v_log_f32 %12, |%12|\n\tv_log_f32 %13, |%13|\n\tv_log_f32 %14, |%14|\n\tv_log_f32 %15, |%15|\n\t"
                 "v_mul_f32 %8, %25, %8\n\tv_mul_f32 %9, %25, %9\n\tv_mul_f32 %10, %25, %10\n\tv_mul_f32 %11, %25, %11\n\t"
                 "v_mul_f32 %12, %25, %12\n\tv_mul_f32 %13, %25, %13\n\tv_mul_f32 %14, %25, %14\n\tv_mul_f32 %15, %25, %15\n\t"
                 "v_exp_f32 %8, %8\n\tv_exp_f32 %9, %9\n\tv_exp_f32 %10, %10\n\tv_exp_f32 %11, %11\n\t"
                 "v_exp_f32 %12, %12\n\tv_exp_f32 %13, %13\n\tv_exp_f32 %14, %14\n\tv_exp_f32 %15, %15\n\t"
                 "v_add_f32 %0, %8, %0\n\tv_add_f32 %1, %9, %1\n\tv_add_f32 %2, %10, %2\n\tv_add_f32 %3, %11, %3\n\t"
                 "v_add_f32 %4, %12, %4\n\tv_add_f32 %5, %13, %5\n\tv_add_f32 %6, %14, %6\n\tv_add_f32 %7, %15, %7"
                 KMC_ROW_OPERANDS(accrow, fa, b), "v"(p));
}

// acc[j][i] += inner(fa[i], fb[j]) for the whole 8 x 8 register tile.
template <int INNER_OP, int INNER_POW>
__device__ __forceinline__ void rank1_update(
    float (&acc)[8][8], const float (&fa)[8], const float (&fb)[8], float p_inner, float diff_sign)
{
    if (INNER_OP == OP_DIFF && INNER_POW == POW_ABS) {
#pragma unroll
        for (int j = 0; j < 8; j++) row_abs_diff(acc[j], fa, fb[j]);
        return;
    }
    if (INNER_OP == OP_DIFF && INNER_POW == POW_SQUARE) {
#pragma unroll
        for (int j = 0; j < 8; j++) row_square_diff(acc[j], fa, fb[j]);
        return;
    }
    if (INNER_OP == OP_DIFF && INNER_POW == POW_POW) {
#pragma unroll
        for (int j = 0; j < 8; j++) row_pow_diff(acc[j], fa, fb[j], p_inner);
        return;
    }
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] += inner_term<INNER_OP, INNER_POW>(fa[i], fb[j], p_inner, diff_sign);
}

// 8 floats of one LDS row: columns [0,4) and [64,68) relative to p.
__device__ __forceinline__ void read_fragment(float (&f)[8], const float *p)
{
    const float4 lo = *reinterpret_cast<const float4 *>(p);
    const float4 hi = *reinterpret_cast<const float4 *>(p + 64);
    f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
    f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
}

// The K walk of an interior tile whose two panels have their rows contiguous and allow 128-bit access (the
// benchmark's storage): the slices go from memory straight into LDS.  global_load_lds_dwordx4 writes the 64 x 16
// bytes of a wave to consecutive LDS addresses, which for these panels are two whole k-rows of 128 floats, so
// the row pitch here is 128 (the 132 of the other loaders only serves their transposing writes).  A lane's
// source address is that of its loader (k-row tid / 32 of the slice, and the one 8 rows further for the
// second copy).  No staging registers and no ds_write: measured on the p = 1 walk at M = N = 30000, K = 1024,
// same box, 29.49 -> 28.86 ms.  The copies are written as instructions because the compiler would make every
// LDS read wait for all of them; it does not count them, so the walk waits for them itself (vmcnt(0) before
// the barrier that publishes a slice) and issues no other vector memory instruction meanwhile.
// `update(fa, fb)` adds the 8 x 8 terms of one k to the caller's accumulators.
template <typename Update>
__device__ __forceinline__ void walk_with_direct_copies(
    TileLoader<LOAD_COL_VEC> &load_a, TileLoader<LOAD_COL_VEC> &load_b, float *lds_a, float *lds_b, int k_slices, int tx, int ty,
    Update &&update)
{
    constexpr int PITCH = BK_TILE_M, SLICE = BK_TILE_K * PITCH;
    static_assert(2 * SLICE + PITCH <= 2 * BK_LDS_SLICE + BK_LDS_PITCH, "the two slices and the pad row fit the staging arrays");
    typedef const __attribute__((address_space(1))) void *global_address;
    typedef __attribute__((address_space(3))) void *lds_address;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const float *src_a = load_a.ptr, *src_b = load_b.ptr;      // of the next slice to copy
    auto copy_slice = [&](int buffer) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            // k-rows 2 wave + 8 j and the next one of the slice
            const unsigned to_a = (unsigned)(unsigned long)(lds_address)(lds_a + buffer * SLICE + (2 * wave + 8 * j) * PITCH);
            const unsigned to_b = (unsigned)(unsigned long)(lds_address)(lds_b + buffer * SLICE + (2 * wave + 8 * j) * PITCH);
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         : : "v"((global_address)(src_a + (i64)(8 * j) * load_a.ld)), "s"(to_a) : "memory", "m0");
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         : : "v"((global_address)(src_b + (i64)(8 * j) * load_b.ld)), "s"(to_b) : "memory", "m0");
        }
        src_a += load_a.step;
        src_b += load_b.step;
    };
    if (k_slices == 0) return;
    // nothing the compiler loaded may be under way beside the copies: it does not know that they count too
    __builtin_amdgcn_s_waitcnt(0x0F70);
    copy_slice(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        if (slice + 1 < k_slices) copy_slice(cur ^ 1);
        const float *sa = lds_a + cur * SLICE + tx * 4;
        const float *sb = lds_b + cur * SLICE + ty * 4;
        float fa0[8], fb0[8], fa1[8], fb1[8];
        read_fragment(fa0, sa);
        read_fragment(fb0, sb);
#pragma unroll 1
        for (int kk = 0; kk < BK_TILE_K; kk += 2) {
            read_fragment(fa1, sa + (kk + 1) * PITCH);
            read_fragment(fb1, sb + (kk + 1) * PITCH);
            update(fa0, fb0);
            read_fragment(fa0, sa + (kk + 2) * PITCH);       // last trip: the other buffer's first row or the pad row, never used
            read_fragment(fb0, sb + (kk + 2) * PITCH);
            update(fa1, fb1);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);      // this wave's copies of the next slice have landed
        __syncthreads();
    }
    load_a.ptr = src_a;      // behind the last slice walked: a caller that walks a contraction in runs goes on from here
    load_b.ptr = src_b;
}

// The K walk for one output tile.  FULL = the tile is interior and K is a
// multiple of the slice depth, so no load needs a predicate; the compiler then
// produces a branch-free steady-state loop.
template <int INNER_OP, int INNER_POW, int LOAD_A, int LOAD_B, bool FULL>
__device__ __forceinline__ void accumulate_tile(
    float (&acc)[8][8], TileLoader<LOAD_A> &load_a, TileLoader<LOAD_B> &load_b,
    float *lds_a, float *lds_b, int k_total, int m_valid, int n_valid, float p_inner, float diff_sign, int tx, int ty)
{
    const int k_slices = (k_total + BK_TILE_K - 1) / BK_TILE_K;
    const int k_tail = k_total - (k_slices - 1) * BK_TILE_K;   // valid k in the last slice
    float stage_a[8], stage_b[8];

    if (k_slices == 0) return;
#ifndef BK_NO_DIRECT_COPIES
    if constexpr (FULL && LOAD_A == LOAD_COL_VEC && LOAD_B == LOAD_COL_VEC) {
        walk_with_direct_copies(load_a, load_b, lds_a, lds_b, k_slices, tx, ty, [&](const float (&fa)[8], const float (&fb)[8]) {
            rank1_update<INNER_OP, INNER_POW>(acc, fa, fb, p_inner, diff_sign);
        });
        return;
    }
#endif
    if (FULL) {
        load_a.load_full(stage_a);
        load_b.load_full(stage_b);
    } else {
        const int kv = k_slices > 1 ? BK_TILE_K : k_tail;
        load_a.load_edge(stage_a, m_valid, kv);
        load_b.load_edge(stage_b, n_valid, kv);
    }
    load_a.store(lds_a, stage_a);
    load_b.store(lds_b, stage_b);
    __syncthreads();

    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) {
            load_a.advance();
            load_b.advance();
            if (FULL) {
                load_a.load_full(stage_a);
                load_b.load_full(stage_b);
            } else {
                const int kv = slice + 2 == k_slices ? k_tail : BK_TILE_K;
                load_a.load_edge(stage_a, m_valid, kv);
                load_b.load_edge(stage_b, n_valid, kv);
            }
        }

        const float *sa = lds_a + cur * BK_LDS_SLICE + tx * 4;
        const float *sb = lds_b + cur * BK_LDS_SLICE + ty * 4;
        // Register double buffer over the 16 k-steps: the fragments of the next
        // step are requested before the 128 VALU operations of the current one
        // are issued.  The loop is kept rolled (two k-steps per trip) on purpose:
        // fully unrolled, the compiler hoists all 64 LDS reads of a slice to the
        // top and needs > 300 registers; rolled, it needs 134 to 142 and three
        // waves fit on each SIMD (a fourth, forced by a register limit of 128,
        // changes nothing measurable).
        float fa0[8], fb0[8], fa1[8], fb1[8];
        read_fragment(fa0, sa);
        read_fragment(fb0, sb);
#pragma unroll 1
        for (int kk = 0; kk < BK_TILE_K; kk += 2) {
            read_fragment(fa1, sa + (kk + 1) * BK_LDS_PITCH);
            read_fragment(fb1, sb + (kk + 1) * BK_LDS_PITCH);
            rank1_update<INNER_OP, INNER_POW>(acc, fa0, fb0, p_inner, diff_sign);
            // On the last trip this reads row 16: the first row of the other
            // buffer or the pad row.  The values are never used; reading them
            // unconditionally keeps the loop free of register copies.
            read_fragment(fa0, sa + (kk + 2) * BK_LDS_PITCH);
            read_fragment(fb0, sb + (kk + 2) * BK_LDS_PITCH);
            rank1_update<INNER_OP, INNER_POW>(acc, fa1, fb1, p_inner, diff_sign);
        }

        if (has_next) {
            load_a.store(lds_a + (cur ^ 1) * BK_LDS_SLICE, stage_a);
            load_b.store(lds_b + (cur ^ 1) * BK_LDS_SLICE, stage_b);
        }
        __syncthreads();
    }
}

// Epilogue on the register tile: outer power, epsilon mask, kernel function and
// the diagonal regularisation (include/build_a_kernel.cuh:374-447).  Lane
// (tx, ty) holds acc[j][i] for n = n0 + ty*4 + (j&3) + (j>>2)*64 and
// m = m0 + tx*4 + (i&3) + (i>>2)*64.
__device__ __forceinline__ void finish_tile(
    float (&acc)[8][8], const BuildKernelArgs &args, int batch, int m0, int n0, int tx, int ty)
{
    const int outer_power = args.outer_power;
    const int kernel_type = args.kernel_type;
    float p_outer = 0.0f, neg_gamma = 0.0f, regularization = 0.0f;
    if (outer_power == POW_POW) {
        p_outer = args.p_outer ? args.p_outer[batch * args.p_outer_bs] : args.p_outer_value;
    }
    if (kernel_type != KERNEL_NONE) {
        const float bw = args.bandwidth ? args.bandwidth[batch * args.bandwidth_bs] : args.bandwidth_value;
        neg_gamma = kernel_neg_gamma(kernel_type, bw);
        regularization = args.regularization ? args.regularization[batch * args.regularization_bs]
                                             : args.regularization_value;
    }
    const float epsilon = args.epsilon;
    // One uniform branch per tile and step, not per element: with the switch inside the
    // loops the compiler keeps it there, and 64 branch chains per lane cost a quarter
    // of the run time of a store-bound (small K) problem.
    auto for_each = [&](auto &&f) {
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[j][i] = f(acc[j][i]);
    };
    switch (outer_power) {
    case POW_ABS: for_each([](float v) { return __builtin_fabsf(v); }); break;
    case POW_SQUARE: for_each([](float v) { return v * v; }); break;
    case POW_SQRT: for_each([](float v) { return __builtin_amdgcn_sqrtf(v); }); break;
    case POW_POW: for_each([p_outer](float v) { return exp2f(p_outer * log2f(v)); }); break;
    default: break;
    }
    if (kernel_type != KERNEL_NONE)
        for_each([epsilon, neg_gamma](float v) { return expf((v < epsilon ? 0.0f : v) * neg_gamma); });
    // include/build_a_kernel.cuh:429-447: the diagonal is replaced, not incremented.
    if (kernel_type != KERNEL_NONE && regularization != 0.0f) {
        const float diagonal_value = 1.0f + regularization;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int n_global = n0 + ty * 4 + (j & 3) + (j >> 2) * 64;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int m_global = m0 + tx * 4 + (i & 3) + (i >> 2) * 64;
                if (args.reg_off_x + m_global == args.reg_off_y + n_global) acc[j][i] = diagonal_value;
            }
        }
    }
}

// Workgroup -> tile.  The hardware deals consecutive workgroup ids round-robin
// over the 8 XCDs, each with its own L2, so XCD x runs ids x, x+8, x+16, ...
// The tile order walks the output in bands of 64 tiles along n, n fastest:
// within a band XCD x therefore owns the 8 n-tiles x, x+8, ..., x+56 and sweeps
// m.  The ~100 workgroups resident on an XCD at any time cover roughly 8 x 12
// tiles and share their A and B panels through that XCD's L2, while ids are
// still handed out in one global order (no XCD can run dry early).  Band
// heights are rounded up to a multiple of 8 to keep that ownership in the last
// band; the padding workgroups get `false` and exit at once.  The host drops the
// rounding for problems of few n tiles, where it would add many such workgroups.
__device__ __forceinline__ bool tile_of_workgroup(const BuildKernelArgs &args, int &tile_m, int &tile_n)
{
    // Batches rotate the order by one: the hardware derives the XCD from the launch-wide
    // workgroup id, which is blockIdx.x modulo 8 for every batch when the grid width is a
    // multiple of 8, so without the rotation a batch of problems of 8 tiles each would
    // run every tile n on a single XCD.  The residue classes modulo 8, and with them the ownership
    // described above, survive the rotation.
    const int rotated = blockIdx.x + blockIdx.y % gridDim.x;
    const int linear = rotated >= (int)gridDim.x ? rotated - (int)gridDim.x : rotated;
    if (args.symmetric) {
        // Symmetric result: the ids count through the tiles on and below the diagonal, row r
        // of the triangle starting at id r (r + 1) / 2.  (In the band order half the
        // workgroups would be empty and XCD x would own the tile rows n = x mod 8, which have
        // different lengths: 80 tiles for XCD 0 and 52 for XCD 7 at 32 x 32 tiles, which then
        // took as long as computing every tile; at 235 x 235 tiles the band order cost 10 %.)
        int row = (int)((sqrtf(8.0f * (float)linear + 1.0f) - 1.0f) * 0.5f);
        while (row * (row + 1) / 2 > linear) row--;
        while ((row + 1) * (row + 2) / 2 <= linear) row++;
        tile_m = row;
        tile_n = linear - row * (row + 1) / 2;
        return true;
    }
    const int band_tiles = BK_BAND_N * args.tiles_m;
    const int band = linear / band_tiles;
    const int band_height = min(BK_BAND_N, args.tiles_n_padded - band * BK_BAND_N);
    const int in_band = linear - band * band_tiles;
    tile_m = in_band / band_height;
    tile_n = band * BK_BAND_N + in_band % band_height;
    return tile_n < args.tiles_n;
}

// Marker the matrix-core L2 kernel (gram_kernel.hpp) leaves in the first element
// of a tile whose result it does not trust: a quiet NaN with a payload no
// arithmetic produces.  In repair mode the kernel below recomputes exactly the
// marked tiles.
constexpr unsigned BK_REPAIR_MARKER = 0x7fc5a5a5u;

// Stores of one finished 128 x 128 register tile (layout of finish_tile): 16 pieces of 4 consecutive m
// per lane, and for a symmetric result the same values again at C(n, m).  `lds_a` / `lds_b` are the
// staging arrays of the K walk, idle by now (the walk ends with a barrier).  `distrusted` (uniform over
// the workgroup; kernels whose tiles the direct kernel may have to recompute) stamps BK_REPAIR_MARKER
// into the tile's first element and leaves the mirrored copy to the repair launch.
__device__ __forceinline__ void store_tile(
    const float (&acc)[8][8], const BuildKernelArgs &args, int batch, int tile_m, int tile_n, int m0, int n0,
    int m_valid, int n_valid, int tx, int ty, int tid, float *lds_a, float *lds_b, bool distrusted)
{
    // Each lane writes 16 pieces of 4 consecutive m.
    float *c_tile = args.c + batch * args.c_bs;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
        if (n_local >= n_valid) continue;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int m_local = tx * 4 + h * 64;
            float *dst = c_tile + (i64)(n0 + n_local) * args.c_ld + m0 + m_local;
            float first = acc[j][4 * h];
            if (distrusted && j == 0 && h == 0 && tid == 0) first = __uint_as_float(BK_REPAIR_MARKER);
            if (args.c_vec && m_local + 3 < m_valid) {
                *reinterpret_cast<float4 *>(dst) = make_float4(first, acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
            } else {
                if (m_local < m_valid) dst[0] = first;
#pragma unroll
                for (int i = 1; i < 4; i++)
                    if (m_local + i < m_valid) dst[i] = acc[j][4 * h + i];
            }
        }
    }

    // Symmetric result: the same values also belong at C(n, m).
    if (args.symmetric && tile_m != tile_n && !distrusted) {
        if (args.c_vec && m_valid >= BK_TILE_M && n_valid >= BK_TILE_N) {
            // Through LDS (idle after the K walk, which ends with a barrier), a quarter of 32 rows m
            // at a time and the two staging arrays in turn, so that every store instruction of a
            // wave writes two whole 512-byte rows of the mirrored tile; written straight from the
            // registers, where a lane's four consecutive n are the contiguous ones, an instruction
            // covers 16 rows with 64 bytes each, and the mirrored half costs 2 of 16.5 ms.
            static_assert(32 * BK_LDS_PITCH <= 2 * BK_LDS_SLICE + BK_LDS_PITCH, "a quarter fits one staging array");
#pragma unroll
            for (int quarter = 0; quarter < 4; quarter++) {
                float *stage = (quarter & 1) ? lds_b : lds_a;
                // rows 32 quarter .. + 31 are held by the lanes with (tx >> 3) == (quarter & 1) in
                // registers i = 4 (quarter >> 1) .. + 3
                if ((tx >> 3) == (quarter & 1)) {
#pragma unroll
                    for (int ii = 0; ii < 4; ii++) {
                        const int i = (quarter >> 1) * 4 + ii;
                        const int row = (tx & 7) * 4 + ii;
#pragma unroll
                        for (int h = 0; h < 2; h++)
                            *reinterpret_cast<float4 *>(stage + row * BK_LDS_PITCH + ty * 4 + h * 64) =
                                make_float4(acc[4 * h][i], acc[4 * h + 1][i], acc[4 * h + 2][i], acc[4 * h + 3][i]);
                    }
                }
                __syncthreads();
#pragma unroll
                for (int pass = 0; pass < 4; pass++) {
                    const int row = pass * 8 + (tid >> 5);
                    const int column = (tid & 31) * 4;
                    const float4 v = *reinterpret_cast<const float4 *>(stage + row * BK_LDS_PITCH + column);
                    *reinterpret_cast<float4 *>(c_tile + (i64)(m0 + quarter * 32 + row) * args.c_ld + n0 + column) = v;
                }
                // the next quarter uses the other array; the one after next waits at that quarter's barrier
            }
        } else {
            // edge tiles and unaligned results: straight from the registers
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int m_local = tx * 4 + (i & 3) + (i >> 2) * 64;
                if (m_local >= m_valid) continue;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int n_local = ty * 4 + h * 64;
                    float *dst = c_tile + (i64)(m0 + m_local) * args.c_ld + n0 + n_local;
                    if (args.c_vec && n_local + 3 < n_valid) {
                        *reinterpret_cast<float4 *>(dst) =
                            make_float4(acc[4 * h][i], acc[4 * h + 1][i], acc[4 * h + 2][i], acc[4 * h + 3][i]);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            if (n_local + j < n_valid) dst[j] = acc[4 * h + j][i];
                    }
                }
            }
        }
    }
}

// One output tile from start to finish; `lds_a` / `lds_b`: two slices per operand plus one pad row (see the fragment
// prefetch).  The body of the two kernels below.
template <int INNER_OP, int INNER_POW, int LOAD_A, int LOAD_B>
__device__ __forceinline__ void build_kernel_tile(const BuildKernelArgs &args, float *lds_a, float *lds_b)
{
    const int tid = threadIdx.x;
    const int batch = blockIdx.y;
    int tile_m, tile_n;
    if (!tile_of_workgroup(args, tile_m, tile_n)) return;
    const int m0 = tile_m * BK_TILE_M;
    const int n0 = tile_n * BK_TILE_N;
    const int m_valid = args.m - m0;   // rows of A that exist from m0 on (may exceed 128)
    const int n_valid = args.n - n0;
    const int tx = tid & 15;
    const int ty = tid >> 4;

    if (args.repair_only) {
        const float first = args.c[batch * args.c_bs + (i64)n0 * args.c_ld + m0];
        if (__float_as_uint(first) != BK_REPAIR_MARKER) return;   // uniform over the workgroup
    }

    float p_inner = 0.0f;
    if (INNER_POW == POW_POW) {
        p_inner = args.p_inner ? args.p_inner[batch * args.p_inner_bs] : args.p_inner_value;
    }

    TileLoader<LOAD_A> load_a;
    TileLoader<LOAD_B> load_b;
    load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
    load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);

    float acc[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;

    const int k_here = args.k_total > 0 ? min(args.k, args.k_total - batch * args.k) : args.k;
    if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && k_here % BK_TILE_K == 0) {
        accumulate_tile<INNER_OP, INNER_POW, LOAD_A, LOAD_B, true>(
            acc, load_a, load_b, lds_a, lds_b, k_here, m_valid, n_valid, p_inner, args.diff_sign, tx, ty);
    } else {
        accumulate_tile<INNER_OP, INNER_POW, LOAD_A, LOAD_B, false>(
            acc, load_a, load_b, lds_a, lds_b, k_here, m_valid, n_valid, p_inner, args.diff_sign, tx, ty);
    }

    // What the epilogue derives from the lane's position is derived here, from a copy of the lane id that the
    // compiler cannot see through: otherwise it computes store addresses before the walk and, in the variant
    // held to 128 registers, parks them in scratch memory for the walk's duration.
    int tid_after = tid;
    asm volatile("" : "+v"(tid_after));
    const int tx_after = tid_after & 15, ty_after = tid_after >> 4;

    finish_tile(acc, args, batch, m0, n0, tx_after, ty_after);

    store_tile(acc, args, batch, tile_m, tile_n, m0, n0, m_valid, n_valid, tx_after, ty_after, tid_after, lds_a, lds_b, false);
}

template <int INNER_OP, int INNER_POW, int LOAD_A, int LOAD_B>
__global__ __launch_bounds__(BK_THREADS) void build_kernel(const BuildKernelArgs args)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    build_kernel_tile<INNER_OP, INNER_POW, LOAD_A, LOAD_B>(args, lds_a, lds_b);
}

// The same kernel for panels with contiguous rows (both loaders LOAD_COL_VEC), compiled for four waves per SIMD.
// Interior tiles of such panels take the walk with direct copies, whose loop needs no staging registers and fits
// the 128 registers of four waves; what spills (about 20 registers) sits in the edge loaders and the epilogue.
// Measured on that walk at M = N = 30000, K = 1024, same box: 28.13 ms at four waves, 28.49 at three, 30.51 at two;
// the product kernels p = 1 29.7 against 30.1 .. 30.5 ms without direct copies, p = 2 31.6 against 32.6.  A launch
// that is bound by its stores (K = 64: 0.68 against 0.66 ms) keeps the three-wave kernel; the host decides by K
// (DIRECT_FOUR_WAVES_MIN_K of host/dispatch_rules.hpp).
template <int INNER_OP, int INNER_POW>
__global__ __launch_bounds__(BK_THREADS, 4) void build_kernel_four_waves(const BuildKernelArgs args)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    build_kernel_tile<INNER_OP, INNER_POW, LOAD_COL_VEC, LOAD_COL_VEC>(args, lds_a, lds_b);
}

}  // namespace kmc
