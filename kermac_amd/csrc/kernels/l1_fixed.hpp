// Opt-in fixed-point path for sums of absolute differences (the L1 norm, Laplace-L1):
//
//   sum_k |b[n,k] - a[m,k]|  =  2^-s * sum_k | qb[n,k] - qa[m,k] |,   q = round(x * 2^s) + 2^(BITS-1)
//
// with the right-hand sum on unsigned integers: v_sad_u32 adds |x - y| to an accumulator in ONE
// instruction where fp32 needs two (subtract, add |x|), and integer sums are exact.  The reference
// has no such path (include/build_a_kernel.cuh:339-370 is fp32 only).  What is lost is the rounding
// of the operands to a common grid: one scale 2^s per batch entry, chosen from the largest magnitude
// in both panels so that every |q - 2^(BITS-1)| <= 2^(BITS-1) - 1.  Each operand is off by at most
// half a grid step, each term by at most one, the sum over K terms by at most K steps -- a bound,
// not an estimate.  Therefore every workgroup checks its own tile: an element whose sum of K terms
// is below K / tolerance steps is not trusted; the workgroup stamps BK_REPAIR_MARKER into the
// tile's first element and the host launches the direct kernel (build_kernel.hpp) in repair mode
// right behind, which recomputes exactly the stamped tiles in fp32 (near-duplicate points, and
// everything when outliers stretch the grid).  Trusted elements carry a relative error below
// `tolerance` (8e-6 unless the caller says otherwise), and on spread-out data far less than the
// fp32 kernel's own rounding (measured 1.7e-7 against 1.5e-6 at K = 1024 on N(0,1) data).
//
// BITS follows the contraction: an accumulator holds 2^(32-BITS) terms of up to 2^BITS - 2 steps, so
// K <= 64 gets 26 bits, K <= 256 24 bits, longer contractions 22 bits and 1024 terms per
// accumulator; after every 1024 terms the sums move into the result (as fp32 partial sums, read
// back and added to after the next 1024).
//
// Steps on the stream (host side: l1_fixed_inst.hip): clear the header, largest magnitude of a and of
// b (l1_fixed_range), a sample of tiles that predicts what share of them will be trusted
// (l1_fixed_sample), both operands to the grid in one layout -- rows contiguous, rows padded to 128
// and k to 16 with the image of zero, so the walk has no edges and needs one loader
// (l1_fixed_convert) -- the walk (l1_fixed_kernel), and the repair launch.
#pragma once

#include "build_kernel.hpp"

namespace kmc {

// Per batch entry, 16 words at the start of the workspace.
struct L1FixedHeader {
    unsigned max_bits;        // bits of the largest |x| in a and b (a NaN or an infinity compares above every number)
    unsigned sampled;         // pairs sampled
    unsigned sampled_below;   // of them, those below the trust threshold
    unsigned sampled_tiles;         // 128 x 128 tiles they were sampled from
    unsigned sampled_tiles_below;   // of them, those that showed such a pair
    unsigned unused[11];
};

// What the sample says: true when the walk would be wasted.  A tile with one element below the threshold is
// recomputed whole, and the walk takes 0.87 of the direct kernel's time, so the route pays while fewer than
// one tile in eight is recomputed.  The share of such tiles is estimated two ways.  Pairs below the threshold
// that are spread evenly (density d) sit in 1 - exp(-16384 d) of the tiles -- one such pair in 100000 is
// already one tile in seven.  Pairs packed into few tiles (points stored cluster by cluster: the blocks on the
// diagonal) sit in the share of sampled tiles that showed one.  Which it is tells the number of sampled tiles
// with such a pair: spread evenly, `below` pairs land in tiles (1 - exp(-below / tiles)) different ones,
// packed, in far fewer.
__device__ __forceinline__ bool l1_fixed_left_to_the_direct_kernel(const L1FixedHeader &header)
{
    if (header.sampled_below == 0u) return false;
    const float pairs = (float)header.sampled, below = (float)header.sampled_below;
    const float tiles = (float)header.sampled_tiles, tiles_below = (float)header.sampled_tiles_below;
    const bool spread = tiles_below >= 0.7f * tiles * (1.0f - __expf(-below / tiles));
    const float share = spread ? 1.0f - __expf(-(float)(BK_TILE_M * BK_TILE_N) * below / pairs) : tiles_below / tiles;
    return share > 0.125f;
}

// The grid of one batch entry, derived from the header by every kernel that needs it.
struct L1FixedGrid {
    float scale;       // 2^s
    float inv_scale;   // 2^-s
    bool usable;       // false: data that is not finite, or all zero / denormal: the direct kernel decides
};

__device__ __forceinline__ L1FixedGrid l1_fixed_grid(unsigned max_bits, int bits)
{
    L1FixedGrid g;
    const int exponent = (int)(max_bits >> 23) - 127;            // largest |x| = 1.f * 2^exponent
    g.usable = max_bits < 0x7f800000u && exponent > -100;
    // |x| < 2^(exponent + 1): 2^s = 2^(bits - 2 - exponent) puts every |x| 2^s below 2^(bits - 1).  The largest
    // may still round up to 2^(bits - 1) itself; then the grid is made one step coarser.
    int s = bits - 2 - exponent;
    s = s > 120 ? 120 : s;
    float scale = __builtin_ldexpf(1.0f, s);
    if (g.usable && __builtin_rintf(__uint_as_float(max_bits) * scale) > (float)((1 << (bits - 1)) - 1)) {
        scale *= 0.5f;
        s -= 1;
    }
    g.scale = scale;
    g.inv_scale = __builtin_ldexpf(1.0f, -s);
    return g;
}

__device__ __forceinline__ int l1_fixed_bits(int k)
{
    return k <= 64 ? 26 : k <= 256 ? 24 : 22;
}

struct L1FixedPanel {
    const float *x; i64 ld, bs;   // the operand as the caller holds it
    int majorness;                // 0: rows contiguous (k strided by ld), 1: k contiguous
    int rows;
    unsigned *q; i64 q_ld, q_bs;  // its image: q[l * q_bs + k * q_ld + row], rows padded to 128, k to 16
};

struct L1FixedArgs {
    BuildKernelArgs kernel;       // m, n, k, l, c, epilogue; a and b are not read
    L1FixedPanel a, b;
    L1FixedHeader *header;        // [l]
    int bits;
    int k_padded;
    float tolerance;              // relative error a trusted element may carry
    int sample_tiles;             // per batch entry
};

constexpr int L1F_THREADS = 256;
constexpr int L1F_TERMS_PER_ACCUMULATOR = 1024;   // at 22 bits

__global__ __launch_bounds__(L1F_THREADS) void l1_fixed_clear(L1FixedHeader *header, int l)
{
    const int i = blockIdx.x * L1F_THREADS + threadIdx.x;
    if (i < l * 16) reinterpret_cast<unsigned *>(header)[i] = 0u;
}

// Largest magnitude of one panel per batch entry: blockIdx.y = batch entry, the workgroups of a
// batch entry stride over the lines along the contiguous direction.
__global__ __launch_bounds__(L1F_THREADS) void l1_fixed_range(const L1FixedPanel panel, int k, L1FixedHeader *header)
{
    const int batch = blockIdx.y;
    const float *x = panel.x + batch * panel.bs;
    const int contiguous = panel.majorness == 0 ? panel.rows : k;
    const int lines = panel.majorness == 0 ? k : panel.rows;
    unsigned largest = 0u;
    for (int line = blockIdx.x; line < lines; line += gridDim.x) {
        const float *p = x + (i64)line * panel.ld;
        // eight loads under way per lane: a lane that waits for every value in turn reads a line of 30000 floats
        // at a quarter of the memory's rate
        for (int i = threadIdx.x; i < contiguous; i += 8 * L1F_THREADS) {
            unsigned bits[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int at = i + u * L1F_THREADS;
                bits[u] = at < contiguous ? __float_as_uint(p[at]) & 0x7fffffffu : 0u;
            }
#pragma unroll
            for (int u = 0; u < 8; u++) largest = bits[u] > largest ? bits[u] : largest;
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const unsigned other = (unsigned)__shfl_xor((int)largest, offset);
        largest = other > largest ? other : largest;
    }
    if ((threadIdx.x & 63) == 0 && largest != 0u) atomicMax(&header[batch].max_bits, largest);
}

__device__ __forceinline__ float l1_fixed_element(const L1FixedPanel &panel, int batch, int row, int kk)
{
    const float *x = panel.x + batch * panel.bs;
    return panel.majorness == 0 ? x[(i64)kk * panel.ld + row] : x[(i64)row * panel.ld + kk];
}

// A sample of the result, summed in fp32 from the operands as the caller holds them: how much of it would not be
// trusted.  A workgroup takes one 128 x 128 tile (blockIdx.x counts the sampled tiles of a batch entry,
// blockIdx.y the batch entries), 16 consecutive rows of a and 16 of b from it, and a lane sums one of their 256
// pairs over all of k; the rows pass through LDS in chunks of 128 k, loaded along whichever direction is
// contiguous.  The conversion and the walk look at the counts before they do anything.
constexpr int L1F_SAMPLE_ROWS = 16;
constexpr int L1F_SAMPLE_CHUNK = 128;
__global__ __launch_bounds__(L1F_THREADS) void l1_fixed_sample(const L1FixedArgs args)
{
    __shared__ float rows_a[L1F_SAMPLE_CHUNK][L1F_SAMPLE_ROWS + 1];      // + 1: no bank is hit twice whichever way the rows are loaded
    __shared__ float rows_b[L1F_SAMPLE_CHUNK][L1F_SAMPLE_ROWS + 1];
    __shared__ unsigned below_in_tile;
    const int batch = blockIdx.y;
    const int t = threadIdx.x;
    const L1FixedGrid grid = l1_fixed_grid(args.header[batch].max_bits, args.bits);
    if (!grid.usable) return;
    if (t == 0) below_in_tile = 0u;
    unsigned h = (unsigned)blockIdx.x * 2654435761u + 0x9e3779b9u * (unsigned)(batch + 1);
    h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 13;
    const int m0 = (int)(h % (unsigned)((args.kernel.m + BK_TILE_M - 1) / BK_TILE_M)) * BK_TILE_M + (int)((h >> 20) & 7u) * L1F_SAMPLE_ROWS;
    h = h * 0x7feb352du + 0x1234567u; h ^= h >> 16;
    const int n0 = (int)(h % (unsigned)((args.kernel.n + BK_TILE_N - 1) / BK_TILE_N)) * BK_TILE_N + (int)((h >> 20) & 7u) * L1F_SAMPLE_ROWS;
    // rows beyond the panel repeat its last row: a pair counted twice biases nothing that matters here
    const int row_a = args.a.majorness == 0 ? t % L1F_SAMPLE_ROWS : t / L1F_SAMPLE_ROWS;
    const int k_a = args.a.majorness == 0 ? t / L1F_SAMPLE_ROWS : t % L1F_SAMPLE_ROWS;
    const int row_b = args.b.majorness == 0 ? t % L1F_SAMPLE_ROWS : t / L1F_SAMPLE_ROWS;
    const int k_b = args.b.majorness == 0 ? t / L1F_SAMPLE_ROWS : t % L1F_SAMPLE_ROWS;
    const int m = min(m0 + row_a, args.kernel.m - 1), n = min(n0 + row_b, args.kernel.n - 1);
    const int i = t % L1F_SAMPLE_ROWS, j = t / L1F_SAMPLE_ROWS;      // this lane's pair: row i of a, row j of b
    float sum = 0.0f;
    for (int k0 = 0; k0 < args.kernel.k; k0 += L1F_SAMPLE_CHUNK) {
        float va[L1F_SAMPLE_CHUNK / 16], vb[L1F_SAMPLE_CHUNK / 16];
#pragma unroll
        for (int u = 0; u < L1F_SAMPLE_CHUNK / 16; u++) {
            const int ka = k0 + k_a + 16 * u, kb = k0 + k_b + 16 * u;
            va[u] = ka < args.kernel.k ? l1_fixed_element(args.a, batch, m, ka) : 0.0f;
            vb[u] = kb < args.kernel.k ? l1_fixed_element(args.b, batch, n, kb) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < L1F_SAMPLE_CHUNK / 16; u++) {
            rows_a[k_a + 16 * u][row_a] = va[u];
            rows_b[k_b + 16 * u][row_b] = vb[u];
        }
        __syncthreads();
#pragma unroll 8
        for (int q = 0; q < L1F_SAMPLE_CHUNK; q++) sum += __builtin_fabsf(rows_b[q][j] - rows_a[q][i]);
    }
    const float threshold = (float)args.kernel.k / args.tolerance * grid.inv_scale;
    if (!(sum >= threshold)) atomicAdd(&below_in_tile, 1u);
    __syncthreads();
    if (t == 0) {
        atomicAdd(&args.header[batch].sampled, (unsigned)L1F_THREADS);
        atomicAdd(&args.header[batch].sampled_tiles, 1u);
        if (below_in_tile > 0u) {
            atomicAdd(&args.header[batch].sampled_below, below_in_tile);
            atomicAdd(&args.header[batch].sampled_tiles_below, 1u);
        }
    }
}

__device__ __forceinline__ unsigned l1_fixed_quantize(float x, const L1FixedGrid &grid, int bits)
{
    return (unsigned)((int)__builtin_rintf(x * grid.scale) + (1 << (bits - 1)));
}

// One operand onto the grid.  A workgroup converts a block of 64 k x 64 rows (blockIdx.x over the
// blocks of rows, blockIdx.y over those of k, blockIdx.z = batch entry); with k contiguous in
// the source the block goes through LDS so that reads and writes are both along contiguous lines.
// Rows and k beyond the panel become the image of zero.
__global__ __launch_bounds__(L1F_THREADS) void l1_fixed_convert(const L1FixedPanel panel, int k, int k_padded, int bits,
                                                                const L1FixedHeader *header)
{
    __shared__ float block[64][65];
    const int batch = blockIdx.z;
    if (l1_fixed_left_to_the_direct_kernel(header[batch])) return;       // the walk will not read the image
    const L1FixedGrid grid = l1_fixed_grid(header[batch].max_bits, bits);
    const int row0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
    const int fast = threadIdx.x & 63, slow = threadIdx.x >> 6;       // 64 x 4 lanes
    const float *x = panel.x + batch * panel.bs;
    unsigned *q = panel.q + batch * panel.q_bs;
    const unsigned zero = 1u << (bits - 1);
    if (panel.majorness == 0) {
        const int row = row0 + fast;
#pragma unroll 4
        for (int i = slow; i < 64; i += 4) {
            const int kk = k0 + i;
            if (kk >= k_padded) break;
            unsigned value = zero;
            if (grid.usable && row < panel.rows && kk < k) value = l1_fixed_quantize(x[(i64)kk * panel.ld + row], grid, bits);
            q[(i64)kk * panel.q_ld + row] = value;
        }
    } else {
#pragma unroll 4
        for (int i = slow; i < 64; i += 4) {
            const int row = row0 + i, kk = k0 + fast;
            block[i][fast] = (row < panel.rows && kk < k) ? x[(i64)row * panel.ld + kk] : 0.0f;
        }
        __syncthreads();
        const int row = row0 + fast;
#pragma unroll 4
        for (int i = slow; i < 64; i += 4) {
            const int kk = k0 + i;
            if (kk >= k_padded) break;
            q[(i64)kk * panel.q_ld + row] = grid.usable ? l1_fixed_quantize(block[fast][i], grid, bits) : zero;
        }
    }
}

// acc[i] += |fa[i] - b| for one row of the register tile, on unsigned integers.
__device__ __forceinline__ void row_sad(unsigned (&accrow)[8], const float (&fa)[8], float b)
{
    asm volatile("v_sad_u32 %0, %8, %16, %0\n\tv_sad_u32 %1, %9, %16, %1\n\tv_sad_u32 %2, %10, %16, %2\n\t"
                 "v_sad_u32 %3, %11, %16, %3\n\tv_sad_u32 %4, %12, %16, %4\n\tv_sad_u32 %5, %13, %16, %5\n\t"
                 "v_sad_u32 %6, %14, %16, %6\n\tv_sad_u32 %7, %15, %16, %7"
                 : "+v"(accrow[0]), "+v"(accrow[1]), "+v"(accrow[2]), "+v"(accrow[3]), "+v"(accrow[4]), "+v"(accrow[5]),
                   "+v"(accrow[6]), "+v"(accrow[7])
                 : "v"(fa[0]), "v"(fa[1]), "v"(fa[2]), "v"(fa[3]), "v"(fa[4]), "v"(fa[5]), "v"(fa[6]), "v"(fa[7]), "v"(b));
}

// The walk: tiles, tile order, direct copies into LDS, fragment reads and stores of build_kernel (the images
// are laid out like panels with contiguous rows, padded, so every tile is an interior one), with the grid
// words travelling as floats untouched.
// Four waves per SIMD: the compiler's own choice is 164 registers, set by the epilogue, not the walk, and three waves;
// within 128 it spills 180 bytes per lane outside the walk, and the launch is 1.4 % faster
// (M = N = 30000, K = 1024, same box: 26.7 -> 26.3 ms).
#ifndef L1F_MIN_WAVES
#define L1F_MIN_WAVES 4
#endif
__global__ __launch_bounds__(BK_THREADS, L1F_MIN_WAVES) void l1_fixed_kernel(const L1FixedArgs fixed)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    const BuildKernelArgs &args = fixed.kernel;
    const int tid = threadIdx.x;
    const int batch = blockIdx.y;
    int tile_m, tile_n;
    if (!tile_of_workgroup(args, tile_m, tile_n)) return;
    const int m0 = tile_m * BK_TILE_M, n0 = tile_n * BK_TILE_N;
    const int m_valid = args.m - m0, n_valid = args.n - n0;
    const int tx = tid & 15, ty = tid >> 4;
    float *c_tile = args.c + batch * args.c_bs;

    const L1FixedHeader header = fixed.header[batch];
    const L1FixedGrid grid = l1_fixed_grid(header.max_bits, fixed.bits);
    if (!grid.usable || l1_fixed_left_to_the_direct_kernel(header)) {
        // nothing here would be trusted, or too little to pay for the walk: leave the whole tile to the repair launch
        if (tid == 0) c_tile[(i64)n0 * args.c_ld + m0] = __uint_as_float(BK_REPAIR_MARKER);
        return;
    }

    TileLoader<LOAD_COL_VEC> load_a, load_b;
    load_a.init(reinterpret_cast<const float *>(fixed.a.q + batch * fixed.a.q_bs), fixed.a.q_ld, m0, tid);
    load_b.init(reinterpret_cast<const float *>(fixed.b.q + batch * fixed.b.q_bs), fixed.b.q_ld, n0, tid);

    // One set of 64 registers holds the integer sums during a run of terms and, between runs and after
    // the last one, the same sums as fp32 bits.
    unsigned acc[8][8];
    const int slices_per_sum = (1 << (32 - fixed.bits)) / BK_TILE_K;
    const int k_slices = fixed.k_padded / BK_TILE_K;
    for (int first = 0; first < k_slices; first += slices_per_sum) {
        const int slices = min(slices_per_sum, k_slices - first);
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[j][i] = 0u;
        walk_with_direct_copies(load_a, load_b, lds_a, lds_b, slices, tx, ty, [&](const float (&fa)[8], const float (&fb)[8]) {
#pragma unroll
            for (int j = 0; j < 8; j++) row_sad(acc[j], fa, fb[j]);
        });
        // This run of terms as fp32, on top of the runs before it, which wait in the result.
        const bool add_earlier = first > 0;
        const bool more_to_come = first + slices < k_slices;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int m_local = tx * 4 + h * 64;
                float *spot = c_tile + (i64)(n0 + n_local) * args.c_ld + m0 + m_local;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float sum = (float)acc[j][4 * h + i] * grid.inv_scale;
                    if (add_earlier || more_to_come) {
                        const bool exists = n_local < n_valid && m_local + i < m_valid;
                        if (add_earlier && exists) sum += spot[i];
                        if (more_to_come && exists) spot[i] = sum;
                    }
                    acc[j][4 * h + i] = __float_as_uint(sum);
                }
            }
        }
    }
    float result[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) result[j][i] = __uint_as_float(acc[j][i]);
    // What the epilogue derives from the lane's position is derived here, from a copy of the lane id that the
    // compiler cannot see through: otherwise it computes the store addresses before the walk and parks them in
    // scratch memory for its duration (27 dwords per lane, written and read back by every tile).
    int tid_after = tid;
    asm volatile("" : "+v"(tid_after));
    const int tx_after = tid_after & 15, ty_after = tid_after >> 4;

    // Trust: an element is off by at most K grid steps.
    const float threshold = (float)args.k / fixed.tolerance * grid.inv_scale;
    int distrust = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int n_local = ty_after * 4 + (j & 3) + (j >> 2) * 64;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int m_local = tx_after * 4 + (i & 3) + (i >> 2) * 64;
            if (n_local < n_valid && m_local < m_valid && !(result[j][i] >= threshold)) distrust = 1;
        }
    }
    const bool distrusted = __syncthreads_or(distrust) != 0;
    finish_tile(result, args, batch, m0, n0, tx_after, ty_after);
    store_tile(result, args, batch, tile_m, tile_n, m0, n0, m_valid, n_valid, tx_after, ty_after, tid_after, lds_a, lds_b, distrusted);
}

}  // namespace kmc
