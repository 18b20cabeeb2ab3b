// What one MI355X issues for the instruction mixes of the cdist inner loops, with nothing but
// registers involved: the rank-1 updates of kmc::build_kernel (kermac_amd/csrc/kernels/build_kernel.hpp:
// row_abs_diff for p = 1, row_square_diff for p = 2, row_pow_diff for a fractional p) and of
// kmc::l1_fixed_kernel (the fixed-point p = 1 path: one v_sad_u32 per term) run on fragments that never
// change, no LDS, no memory.  The rates printed here are the issue ceilings that bench.py reports
// the cdist kernels against (frac_of_issue_ceiling, issue_floor_ms): a kernel cannot retire its 2
// (p = 1, 2), 5 (fractional p, two of them transcendental) or 1 (fixed point) instructions per
// (m, n, k) faster than this.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         bench_issue_rates.hip -o /tmp/bench_issue_rates
//   /tmp/bench_issue_rates [min_ms]
//   /tmp/bench_issue_rates walk          (second mode, described further down)
//
// Every case is one launch of at least `min_ms` milliseconds (default 3; 30 is the duration of the
// p = 1 cdist launch at M = N = 30000, K = 1024, so the clock the board sustains over such a launch
// shows).  Per case and per number of waves on a SIMD: time, nanoseconds per wave instruction per
// SIMD, lane operations per second for the whole chip, the shader clock during the run (shader
// clock ticks per microsecond of the 100 MHz wall clock), cycles per instruction, and the time the
// M = N = 30000, K = 1024 problem would take at that rate.  The last lines are "key = value" pairs:
// per case the fastest of 2, 3 and 4 waves per SIMD, which is what the vector ALU can do.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "kermac_amd/csrc/kernels/build_kernel.hpp"
#include "kermac_amd/csrc/kernels/build_kernel_scalar_b.hpp"

#define CHECK(x) \
    do { \
        hipError_t e_ = (x); \
        if (e_ != hipSuccess) { \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            return 1; \
        } \
    } while (0)

enum Case { P1_ROWS, P2_ROWS, POW_ROWS, PLAIN_ADD, ABS_ADD, EXP2, LOG2, SAD_U32, CASES };
static const char *case_names[CASES] = {
    "p = 1 rows: 8 v_sub + 8 v_add |x|", "p = 2 rows: 8 v_sub + 8 v_fmac", "p = 1.3 rows: sub, log2, mul, exp2, add",
    "v_add_f32 (4-byte encoding)",        "v_add_f32 |x| (8-byte encoding)", "v_exp_f32", "v_log_f32",
    "v_sad_u32 (|a - b| + c on integers)"};
static const char *case_keys[CASES] = {"p1_rows", "p2_rows", "pow_rows", "v_add_f32", "v_add_f32_abs", "v_exp_f32", "v_log_f32",
                                       "v_sad_u32"};
// vector instructions per (m, n, k) of the case
static const int per_term[CASES] = {2, 2, 5, 1, 1, 1, 1, 1};

template <int CASE>
__global__ __launch_bounds__(1024) void issue(float *out, long long *clocks, int updates, float seed)
{
    float acc[8][8], fa[8], fb[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        fa[j] = seed + 0.25f * j;            // differences stay in 1.25 .. 4.75: no denormals, no infinities
        fb[j] = seed + 3.0f + 0.25f * j;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;
    }
    const long long wall0 = wall_clock64(), tick0 = clock64();
    for (int u = 0; u < updates; u++) {
        if (CASE == P1_ROWS) kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc, fa, fb, 0.0f, 1.0f);
        if (CASE == P2_ROWS) kmc::rank1_update<kmc::OP_DIFF, kmc::POW_SQUARE>(acc, fa, fb, 0.0f, 1.0f);
        if (CASE == POW_ROWS) kmc::rank1_update<kmc::OP_DIFF, kmc::POW_POW>(acc, fa, fb, 1.3f, 1.0f);
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (CASE == PLAIN_ADD) asm volatile("v_add_f32 %0, %1, %0" : "+v"(acc[j][i]) : "v"(fa[i]));
                if (CASE == ABS_ADD) asm volatile("v_add_f32 %0, |%1|, %0" : "+v"(acc[j][i]) : "v"(fa[i]));
                if (CASE == EXP2) asm volatile("v_exp_f32 %0, %1" : "=v"(acc[j][i]) : "v"(fa[i]));
                if (CASE == LOG2) asm volatile("v_log_f32 %0, %1" : "=v"(acc[j][i]) : "v"(fb[i]));
                if (CASE == SAD_U32) asm volatile("v_sad_u32 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(fa[i]), "v"(fb[j]));
            }
    }
    const long long wall1 = wall_clock64(), tick1 = clock64();
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) sum += acc[j][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = wall1 - wall0;
        clocks[1] = tick1 - tick0;
    }
}


// ---- second mode: `bench_issue_rates walk` ------------------------------------------------------------
// The p = 1 walk of kmc::build_kernel at M = N = 30000, K = 1024 with parts of its memory traffic left
// out, to see what each part costs in time and in shader clock (one workgroup from the middle of the
// launch reads both clocks around its walk): global loads, LDS writes, LDS fragment reads, barriers.
// The results of the variants are wrong on purpose; only the product kernel's line is a cdist.
__global__ void fill(float *x, long long n, unsigned seed)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    unsigned h = (unsigned)i * 2654435761u + seed; h ^= h >> 15; h *= 0x846ca68bU; h ^= h >> 16;
    x[i] = (h >> 8) * (1.0f / 8388608.0f) - 1.0f;
}

// NO_GLOBAL: slices after the first reuse the first slice's registers (no HBM/L2 traffic in the walk)
// NO_LDS_READ: fragments are read once per slice instead of once per k
// NO_LDS_WRITE: staging stores skipped after the first slice
template <bool NO_GLOBAL, bool NO_LDS_READ, bool NO_LDS_WRITE, bool NO_BARRIER>
__global__ __launch_bounds__(kmc::BK_THREADS) void walk_variant(const kmc::BuildKernelArgs args, long long *clocks)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    const int tid = threadIdx.x;
    int tile_m, tile_n;
    if (!kmc::tile_of_workgroup(args, tile_m, tile_n)) return;
    const long long wall0 = wall_clock64(), tick0 = clock64();
    const int m0 = tile_m * kmc::BK_TILE_M, n0 = tile_n * kmc::BK_TILE_N;
    const int tx = tid & 15, ty = tid >> 4;
    kmc::TileLoader<kmc::LOAD_COL_VEC> load_a, load_b;
    load_a.init(args.a, args.a_ld, m0, tid);
    load_b.init(args.b, args.b_ld, n0, tid);
    float acc[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;
    const int k_slices = args.k / kmc::BK_TILE_K;
    float stage_a[8], stage_b[8];
    load_a.load_full(stage_a);
    load_b.load_full(stage_b);
    load_a.store(lds_a, stage_a); load_b.store(lds_b, stage_b);
    load_a.store(lds_a + kmc::BK_LDS_SLICE, stage_a); load_b.store(lds_b + kmc::BK_LDS_SLICE, stage_b);
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next && !NO_GLOBAL) {
            load_a.advance(); load_b.advance();
            load_a.load_full(stage_a); load_b.load_full(stage_b);
        }
        const float *sa = lds_a + cur * kmc::BK_LDS_SLICE + tx * 4;
        const float *sb = lds_b + cur * kmc::BK_LDS_SLICE + ty * 4;
        float fa0[8], fb0[8], fa1[8], fb1[8];
        kmc::read_fragment(fa0, sa); kmc::read_fragment(fb0, sb);
        if (NO_LDS_READ) { kmc::read_fragment(fa1, sa + kmc::BK_LDS_PITCH); kmc::read_fragment(fb1, sb + kmc::BK_LDS_PITCH); }
#pragma unroll 1
        for (int kk = 0; kk < kmc::BK_TILE_K; kk += 2) {
            if (!NO_LDS_READ) { kmc::read_fragment(fa1, sa + (kk + 1) * kmc::BK_LDS_PITCH); kmc::read_fragment(fb1, sb + (kk + 1) * kmc::BK_LDS_PITCH); }
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc, fa0, fb0, 0.0f, 1.0f);
            if (!NO_LDS_READ) { kmc::read_fragment(fa0, sa + (kk + 2) * kmc::BK_LDS_PITCH); kmc::read_fragment(fb0, sb + (kk + 2) * kmc::BK_LDS_PITCH); }
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc, fa1, fb1, 0.0f, 1.0f);
        }
        if (has_next && !NO_LDS_WRITE) {
            load_a.store(lds_a + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_a);
            load_b.store(lds_b + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_b);
        }
        if (!NO_BARRIER) __syncthreads();
    }
    const long long wall1 = wall_clock64(), tick1 = clock64();
    float *c_tile = args.c;
    const int m_valid = args.m - m0, n_valid = args.n - n0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
        if (n_local >= n_valid) continue;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int m_local = tx * 4 + h * 64;
            float *dst = c_tile + (kmc::i64)(n0 + n_local) * args.c_ld + m0 + m_local;
            if (m_local + 3 < m_valid)
                *reinterpret_cast<float4 *>(dst) = make_float4(acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
        }
    }
    // a workgroup from the middle of the launch reports its clocks
    if (tid == 0 && blockIdx.x == gridDim.x / 2) { clocks[0] = wall1 - wall0; clocks[1] = tick1 - tick0; }
}


// The same walk on a tile of 128 (m) x 256 (n) per workgroup, 8 x 16 results per lane: one fragment of a meets two
// fragments of b, so a term needs 0.1875 floats from LDS instead of 0.25 and the launch asks the L2s for 43 GB instead
// of 58.  Two waves per SIMD (about 210 registers).  Stores only the first half of n (timing only).
__global__ __launch_bounds__(kmc::BK_THREADS, 2) void walk_wide_tile(const kmc::BuildKernelArgs args, long long *clocks)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b0[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b1[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    const int tid = threadIdx.x;
    // bands of 32 double tiles along n, n fastest: XCD x owns 4 of them
    const int tiles_n2 = (args.tiles_n + 1) / 2, padded = (tiles_n2 + 7) / 8 * 8;
    const int band_tiles = 32 * args.tiles_m;
    const int band = blockIdx.x / band_tiles;
    const int band_height = min(32, padded - band * 32);
    const int in_band = blockIdx.x - band * band_tiles;
    const int tile_m = in_band / band_height, tile_n = band * 32 + in_band % band_height;
    if (tile_n >= tiles_n2) return;
    const long long wall0 = wall_clock64(), tick0 = clock64();
    const int m0 = tile_m * kmc::BK_TILE_M, n0 = tile_n * 2 * kmc::BK_TILE_N;
    const int tx = tid & 15, ty = tid >> 4;
    kmc::TileLoader<kmc::LOAD_COL_VEC> load_a, load_b0, load_b1;
    load_a.init(args.a, args.a_ld, m0, tid);
    load_b0.init(args.b, args.b_ld, n0, tid);
    load_b1.init(args.b, args.b_ld, min(n0 + kmc::BK_TILE_N, (args.tiles_n - 1) * kmc::BK_TILE_N), tid);
    float acc0[8][8], acc1[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc0[j][i] = acc1[j][i] = 0.0f;
    const int k_slices = args.k / kmc::BK_TILE_K;
    float stage_a[8], stage_b0[8], stage_b1[8];
    load_a.load_full(stage_a); load_b0.load_full(stage_b0); load_b1.load_full(stage_b1);
    load_a.store(lds_a, stage_a); load_b0.store(lds_b0, stage_b0); load_b1.store(lds_b1, stage_b1);
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) {
            load_a.advance(); load_b0.advance(); load_b1.advance();
            load_a.load_full(stage_a); load_b0.load_full(stage_b0); load_b1.load_full(stage_b1);
        }
        const float *sa = lds_a + cur * kmc::BK_LDS_SLICE + tx * 4;
        const float *sb0 = lds_b0 + cur * kmc::BK_LDS_SLICE + ty * 4;
        const float *sb1 = lds_b1 + cur * kmc::BK_LDS_SLICE + ty * 4;
        float fa0[8], fb00[8], fb01[8], fa1[8], fb10[8], fb11[8];
        kmc::read_fragment(fa0, sa); kmc::read_fragment(fb00, sb0); kmc::read_fragment(fb01, sb1);
#pragma unroll 1
        for (int kk = 0; kk < kmc::BK_TILE_K; kk += 2) {
            kmc::read_fragment(fa1, sa + (kk + 1) * kmc::BK_LDS_PITCH);
            kmc::read_fragment(fb10, sb0 + (kk + 1) * kmc::BK_LDS_PITCH);
            kmc::read_fragment(fb11, sb1 + (kk + 1) * kmc::BK_LDS_PITCH);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc0, fa0, fb00, 0.0f, 1.0f);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc1, fa0, fb01, 0.0f, 1.0f);
            kmc::read_fragment(fa0, sa + (kk + 2) * kmc::BK_LDS_PITCH);
            kmc::read_fragment(fb00, sb0 + (kk + 2) * kmc::BK_LDS_PITCH);
            kmc::read_fragment(fb01, sb1 + (kk + 2) * kmc::BK_LDS_PITCH);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc0, fa1, fb10, 0.0f, 1.0f);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc1, fa1, fb11, 0.0f, 1.0f);
        }
        if (has_next) {
            load_a.store(lds_a + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_a);
            load_b0.store(lds_b0 + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_b0);
            load_b1.store(lds_b1 + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_b1);
        }
        __syncthreads();
    }
    const long long wall1 = wall_clock64(), tick1 = clock64();
    const int m_valid = args.m - m0;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        const int n_valid = args.n - n0 - half * kmc::BK_TILE_N;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
            if (n_local >= n_valid) continue;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int m_local = tx * 4 + h * 64;
                float *dst = args.c + (kmc::i64)(n0 + half * kmc::BK_TILE_N + n_local) * args.c_ld + m0 + m_local;
                const float (&acc)[8][8] = half ? acc1 : acc0;
                if (m_local + 3 < m_valid)
                    *reinterpret_cast<float4 *>(dst) = make_float4(acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
            }
        }
    }
    if (tid == 0 && blockIdx.x == gridDim.x / 2) { clocks[0] = wall1 - wall0; clocks[1] = tick1 - tick0; }
}

typedef float frag4 __attribute__((ext_vector_type(4)));
struct Fragments {
    frag4 a_lo, a_hi, b0_lo, b0_hi, b1_lo, b1_hi;
};
#define READ_FRAGMENTS(f, pa, pb0, pb1, lo, hi) \
    asm volatile("ds_read_b128 %0, %6 offset:" lo "\n\tds_read_b128 %1, %6 offset:" hi "\n\t" \
                 "ds_read_b128 %2, %7 offset:" lo "\n\tds_read_b128 %3, %7 offset:" hi "\n\t" \
                 "ds_read_b128 %4, %8 offset:" lo "\n\tds_read_b128 %5, %8 offset:" hi \
                 : "=&v"(f.a_lo), "=&v"(f.a_hi), "=&v"(f.b0_lo), "=&v"(f.b0_hi), "=&v"(f.b1_lo), "=&v"(f.b1_hi) \
                 : "v"(pa), "v"(pb0), "v"(pb1) \
                 : "memory")

__device__ __forceinline__ void update_from(float (&acc0)[8][8], float (&acc1)[8][8], const Fragments &f)
{
    const float fa[8] = {f.a_lo.x, f.a_lo.y, f.a_lo.z, f.a_lo.w, f.a_hi.x, f.a_hi.y, f.a_hi.z, f.a_hi.w};
    const float fb0[8] = {f.b0_lo.x, f.b0_lo.y, f.b0_lo.z, f.b0_lo.w, f.b0_hi.x, f.b0_hi.y, f.b0_hi.z, f.b0_hi.w};
    const float fb1[8] = {f.b1_lo.x, f.b1_lo.y, f.b1_lo.z, f.b1_lo.w, f.b1_hi.x, f.b1_hi.y, f.b1_hi.z, f.b1_hi.w};
    kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc0, fa, fb0, 0.0f, 1.0f);
    kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc1, fa, fb1, 0.0f, 1.0f);
}

// The wide tile again with the fragment reads written as instructions and the waits counted by hand: the compiler puts
// s_waitcnt lgkmcnt(0) behind the reads of the next k at the head of the rolled loop (it loses count over the back
// edge), which exposes the LDS latency once per trip; with three waves on a SIMD the others cover it, with two they do not.
__global__ __launch_bounds__(kmc::BK_THREADS, 2) void walk_wide_tile_counted(const kmc::BuildKernelArgs args, long long *clocks)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b0[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b1[2 * kmc::BK_LDS_SLICE + kmc::BK_LDS_PITCH];
    const int tid = threadIdx.x;
    // bands of 32 double tiles along n, n fastest: XCD x owns 4 of them
    const int tiles_n2 = (args.tiles_n + 1) / 2, padded = (tiles_n2 + 7) / 8 * 8;
    const int band_tiles = 32 * args.tiles_m;
    const int band = blockIdx.x / band_tiles;
    const int band_height = min(32, padded - band * 32);
    const int in_band = blockIdx.x - band * band_tiles;
    const int tile_m = in_band / band_height, tile_n = band * 32 + in_band % band_height;
    if (tile_n >= tiles_n2) return;
    const long long wall0 = wall_clock64(), tick0 = clock64();
    const int m0 = tile_m * kmc::BK_TILE_M, n0 = tile_n * 2 * kmc::BK_TILE_N;
    const int tx = tid & 15, ty = tid >> 4;
    kmc::TileLoader<kmc::LOAD_COL_VEC> load_a, load_b0, load_b1;
    load_a.init(args.a, args.a_ld, m0, tid);
    load_b0.init(args.b, args.b_ld, n0, tid);
    load_b1.init(args.b, args.b_ld, min(n0 + kmc::BK_TILE_N, (args.tiles_n - 1) * kmc::BK_TILE_N), tid);
    float acc0[8][8], acc1[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc0[j][i] = acc1[j][i] = 0.0f;
    const int k_slices = args.k / kmc::BK_TILE_K;
    float stage_a[8], stage_b0[8], stage_b1[8];
    load_a.load_full(stage_a); load_b0.load_full(stage_b0); load_b1.load_full(stage_b1);
    load_a.store(lds_a, stage_a); load_b0.store(lds_b0, stage_b0); load_b1.store(lds_b1, stage_b1);
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) {
            load_a.advance(); load_b0.advance(); load_b1.advance();
            load_a.load_full(stage_a); load_b0.load_full(stage_b0); load_b1.load_full(stage_b1);
        }
        const float *sa = lds_a + cur * kmc::BK_LDS_SLICE + tx * 4;
        const float *sb0 = lds_b0 + cur * kmc::BK_LDS_SLICE + ty * 4;
        const float *sb1 = lds_b1 + cur * kmc::BK_LDS_SLICE + ty * 4;
        typedef __attribute__((address_space(3))) void *lds_address;
        unsigned pa = (unsigned)(unsigned long)(lds_address)sa, pb0 = (unsigned)(unsigned long)(lds_address)sb0,
                 pb1 = (unsigned)(unsigned long)(lds_address)sb1;
        Fragments even, odd;
        READ_FRAGMENTS(even, pa, pb0, pb1, "0", "256");
#pragma unroll 1
        for (int kk = 0; kk < kmc::BK_TILE_K; kk += 2) {
            READ_FRAGMENTS(odd, pa, pb0, pb1, "528", "784");
            asm volatile("s_waitcnt lgkmcnt(6)" ::: "memory");
            update_from(acc0, acc1, even);
            READ_FRAGMENTS(even, pa, pb0, pb1, "1056", "1312");     // last trip: a row that is never used
            asm volatile("s_waitcnt lgkmcnt(6)" ::: "memory");
            update_from(acc0, acc1, odd);
            pa += 1056; pb0 += 1056; pb1 += 1056;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (has_next) {
            load_a.store(lds_a + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_a);
            load_b0.store(lds_b0 + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_b0);
            load_b1.store(lds_b1 + (cur ^ 1) * kmc::BK_LDS_SLICE, stage_b1);
        }
        __syncthreads();
    }
    const long long wall1 = wall_clock64(), tick1 = clock64();
    const int m_valid = args.m - m0;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        const int n_valid = args.n - n0 - half * kmc::BK_TILE_N;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
            if (n_local >= n_valid) continue;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int m_local = tx * 4 + h * 64;
                float *dst = args.c + (kmc::i64)(n0 + half * kmc::BK_TILE_N + n_local) * args.c_ld + m0 + m_local;
                const float (&acc)[8][8] = half ? acc1 : acc0;
                if (m_local + 3 < m_valid)
                    *reinterpret_cast<float4 *>(dst) = make_float4(acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
            }
        }
    }
    if (tid == 0 && blockIdx.x == gridDim.x / 2) { clocks[0] = wall1 - wall0; clocks[1] = tick1 - tick0; }
}


// The walk with the panels copied from memory straight into LDS (global_load_lds_dwordx4: a wave writes two
// k-rows of 128 floats, 1 KB, per instruction; no registers, no ds_write; LDS pitch 128 instead of 132) on its own,
// at 4, 3 and 2 waves per SIMD: what the product kernel's interior tiles run (accumulate_tile_direct).  The variants
// further up ("same walk", "no global loads" ...) are the walk through staging registers that other layouts take.
template <int WAVES>
__global__ __launch_bounds__(kmc::BK_THREADS) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void walk_direct_to_lds(const kmc::BuildKernelArgs args, long long *clocks)
{
    constexpr int PITCH = kmc::BK_TILE_M, SLICE = kmc::BK_TILE_K * PITCH;
    __shared__ __attribute__((aligned(16))) float lds_a[2 * SLICE + PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * SLICE + PITCH];
    const int tid = threadIdx.x;
    int tile_m, tile_n;
    if (!kmc::tile_of_workgroup(args, tile_m, tile_n)) return;
    const long long wall0 = wall_clock64(), tick0 = clock64();
    const int m0 = tile_m * kmc::BK_TILE_M, n0 = tile_n * kmc::BK_TILE_N;
    const int tx = tid & 15, ty = tid >> 4;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    typedef const __attribute__((address_space(1))) void *global_address;
    typedef __attribute__((address_space(3))) void *lds_address;
    // copy j of 2 per operand: k-rows 4 * wave + 2 * j + (lane >> 5), 16 bytes number lane & 31 of the row
    const float *src_a[2], *src_b[2];
    int dst[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int k_row = 4 * wave + 2 * j + (lane >> 5);
        src_a[j] = args.a + (kmc::i64)k_row * args.a_ld + m0 + 4 * (lane & 31);
        src_b[j] = args.b + (kmc::i64)k_row * args.b_ld + n0 + 4 * (lane & 31);
        dst[j] = (4 * wave + 2 * j) * PITCH;
    }
    const kmc::i64 step_a = (kmc::i64)kmc::BK_TILE_K * args.a_ld, step_b = (kmc::i64)kmc::BK_TILE_K * args.b_ld;
    auto copy_slice = [&](int buffer) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const unsigned to_a = (unsigned)(unsigned long)(lds_address)(lds_a + buffer * SLICE + dst[j]);
            const unsigned to_b = (unsigned)(unsigned long)(lds_address)(lds_b + buffer * SLICE + dst[j]);
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"((global_address)src_a[j]), "s"(to_a) : "memory", "m0");
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"((global_address)src_b[j]), "s"(to_b) : "memory", "m0");
            src_a[j] += step_a;
            src_b[j] += step_b;
        }
    };
    float acc[8][8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;
    const int k_slices = args.k / kmc::BK_TILE_K;
    copy_slice(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        if (slice + 1 < k_slices) copy_slice(cur ^ 1);
        const float *sa = lds_a + cur * SLICE + tx * 4;
        const float *sb = lds_b + cur * SLICE + ty * 4;
        float fa0[8], fb0[8], fa1[8], fb1[8];
        kmc::read_fragment(fa0, sa); kmc::read_fragment(fb0, sb);
#pragma unroll 1
        for (int kk = 0; kk < kmc::BK_TILE_K; kk += 2) {
            kmc::read_fragment(fa1, sa + (kk + 1) * PITCH); kmc::read_fragment(fb1, sb + (kk + 1) * PITCH);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc, fa0, fb0, 0.0f, 1.0f);
            kmc::read_fragment(fa0, sa + (kk + 2) * PITCH); kmc::read_fragment(fb0, sb + (kk + 2) * PITCH);
            kmc::rank1_update<kmc::OP_DIFF, kmc::POW_ABS>(acc, fa1, fb1, 0.0f, 1.0f);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);      // this wave's copies of the next slice have landed
        __syncthreads();
    }
    const long long wall1 = wall_clock64(), tick1 = clock64();
    const int m_valid = args.m - m0, n_valid = args.n - n0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int n_local = ty * 4 + (j & 3) + (j >> 2) * 64;
        if (n_local >= n_valid) continue;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int m_local = tx * 4 + h * 64;
            float *dst_c = args.c + (kmc::i64)(n0 + n_local) * args.c_ld + m0 + m_local;
            if (m_local + 3 < m_valid)
                *reinterpret_cast<float4 *>(dst_c) = make_float4(acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
        }
    }
    if (tid == 0 && blockIdx.x == gridDim.x / 2) { clocks[0] = wall1 - wall0; clocks[1] = tick1 - tick0; }
}

#define CHECK_VOID(x) \
    do { \
        hipError_t e_ = (x); \
        if (e_ != hipSuccess) { \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            exit(1); \
        } \
    } while (0)

template <typename F>
void run(const char *what, F launch, long long *clocks, int reps)
{
    hipEvent_t e0, e1;
    CHECK_VOID(hipEventCreate(&e0)); CHECK_VOID(hipEventCreate(&e1));
    launch(); CHECK_VOID(hipDeviceSynchronize());
    float best = 1e30f; long long hc[2] = {1, 0};
    for (int r = 0; r < reps; r++) {
        CHECK_VOID(hipEventRecord(e0)); launch(); CHECK_VOID(hipEventRecord(e1)); CHECK_VOID(hipEventSynchronize(e1));
        float ms; CHECK_VOID(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) { best = ms; CHECK_VOID(hipMemcpy(hc, clocks, sizeof hc, hipMemcpyDeviceToHost)); }
    }
    CHECK_VOID(hipGetLastError());
    printf("%-58s %8.3f ms   clock of one mid-launch workgroup %4.0f MHz (its walk %.1f us)\n", what, best,
           (double)hc[1] / ((double)hc[0] / 100.0), hc[0] / 100.0);
    fflush(stdout);
}

int walk_ablations()
{
    const int M = 30000, N = 30000, K = 1024, reps = 4;
    const int Mp = (M + 127) / 128 * 128, Np = (N + 127) / 128 * 128;
    float *a, *b, *c; long long *clocks;
    CHECK(hipMalloc(&a, (size_t)K * Mp * 4)); CHECK(hipMalloc(&b, (size_t)K * Np * 4)); CHECK(hipMalloc(&c, (size_t)N * M * 4));
    CHECK(hipMalloc(&clocks, 16));
    fill<<<(unsigned)(((long long)K * Mp + 255) / 256), 256>>>(a, (long long)K * Mp, 1u);
    fill<<<(unsigned)(((long long)K * Np + 255) / 256), 256>>>(b, (long long)K * Np, 7u);
    CHECK(hipDeviceSynchronize());
    const int tiles_m = Mp / 128, tiles_n = Np / 128, tiles_n_padded = (tiles_n + 7) / 8 * 8;
    const dim3 grid(tiles_m * tiles_n_padded);
    kmc::BuildKernelArgs d = {};
    d.m = M; d.n = N; d.k = K; d.l = 1; d.a = a; d.a_ld = Mp; d.b = b; d.b_ld = Np; d.c = c; d.c_ld = M;
    d.diff_sign = 1.0f; d.c_vec = 1; d.tiles_m = tiles_m; d.tiles_n = tiles_n; d.tiles_n_padded = tiles_n_padded; d.grid_width = grid.x;
    const dim3 scalar_b_grid(((M + kmc::SB_TILE_M - 1) / kmc::SB_TILE_M) * ((N + kmc::SB_TILE_N - 1) / kmc::SB_TILE_N));
    run("product kernel build_kernel_scalar_b<DIFF, ABS> (b in scalar registers)", [&] { kmc::build_kernel_scalar_b<kmc::OP_DIFF, kmc::POW_ABS><<<scalar_b_grid, 256>>>(d, a, b, c); }, clocks, reps);
    run("product kernel build_kernel_four_waves<DIFF, ABS>", [&] { kmc::build_kernel_four_waves<kmc::OP_DIFF, kmc::POW_ABS><<<grid, 256>>>(d); }, clocks, reps);
    run("product kernel at three waves per SIMD, build_kernel<DIFF, ABS>", [&] { kmc::build_kernel<kmc::OP_DIFF, kmc::POW_ABS, kmc::LOAD_COL_VEC, kmc::LOAD_COL_VEC><<<grid, 256>>>(d); }, clocks, reps);
    run("same walk, clocks read (all traffic)", [&] { walk_variant<false, false, false, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("no global loads in the walk", [&] { walk_variant<true, false, false, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("no global loads, no LDS writes", [&] { walk_variant<true, false, true, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("no global loads, no LDS writes, no barriers", [&] { walk_variant<true, false, true, true><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("LDS fragments read once per slice", [&] { walk_variant<false, true, false, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("no global loads, fragments once per slice", [&] { walk_variant<true, true, false, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("nothing but the arithmetic (and barriers)", [&] { walk_variant<true, true, true, false><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("nothing but the arithmetic", [&] { walk_variant<true, true, true, true><<<grid, 256>>>(d, clocks); }, clocks, reps);
    const int tiles_n2 = (tiles_n + 1) / 2;
    const dim3 wide_grid(tiles_m * ((tiles_n2 + 7) / 8 * 8));
    run("tile of 128 x 256, 8 x 16 results per lane, 2 waves per SIMD", [&] { walk_wide_tile<<<wide_grid, 256>>>(d, clocks); }, clocks, reps);
    run("the same with the LDS waits counted by hand", [&] { walk_wide_tile_counted<<<wide_grid, 256>>>(d, clocks); }, clocks, reps);
    run("product walk, panels copied straight into LDS, 4 waves per SIMD", [&] { walk_direct_to_lds<4><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("the same, 3 waves per SIMD", [&] { walk_direct_to_lds<3><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("the same, 2 waves per SIMD", [&] { walk_direct_to_lds<2><<<grid, 256>>>(d, clocks); }, clocks, reps);
    run("product kernel build_kernel_four_waves<DIFF, ABS> again", [&] { kmc::build_kernel_four_waves<kmc::OP_DIFF, kmc::POW_ABS><<<grid, 256>>>(d); }, clocks, reps);
    run("product kernel build_kernel_scalar_b<DIFF, ABS> again", [&] { kmc::build_kernel_scalar_b<kmc::OP_DIFF, kmc::POW_ABS><<<scalar_b_grid, 256>>>(d, a, b, c); }, clocks, reps);
    float direct_element;
    CHECK_VOID(hipMemcpy(&direct_element, c + (size_t)12345 * M + 6789, 4, hipMemcpyDeviceToHost));
    printf("one element from the walk with direct copies %.6f\n", direct_element);
    float got[2];
    CHECK_VOID(hipMemcpy(got, c + (size_t)12345 * M + 6789, 4, hipMemcpyDeviceToHost));
    kmc::build_kernel_four_waves<kmc::OP_DIFF, kmc::POW_ABS><<<grid, 256>>>(d);
    CHECK_VOID(hipMemcpy(got + 1, c + (size_t)12345 * M + 6789, 4, hipMemcpyDeviceToHost));
    printf("one element from the wide tile %.6f, from the product kernel %.6f\n", got[0], got[1]);
    return 0;
}

struct Result {
    double ms, ns_per_instruction, lane_ops_per_s, mhz;
};
static Result results[CASES][5];

template <int CASE>
int measure(float *out, long long *clocks, int waves_per_simd, double min_ms)
{
    // one workgroup of 4 * waves_per_simd waves on every CU: each SIMD holds waves_per_simd of them
    const int cus = 256;
    int updates = (CASE == POW_ROWS || CASE == EXP2 || CASE == LOG2) ? 1500 : 6000;
    hipEvent_t start, stop;
    CHECK(hipEventCreate(&start));
    CHECK(hipEventCreate(&stop));
    issue<CASE><<<cus, 256 * waves_per_simd>>>(out, clocks, 10, 1.0f);
    CHECK(hipDeviceSynchronize());
    float best = 1e30f;
    long long best_clocks[2] = {1, 0};
    // a first launch sizes the run; then three launches of at least min_ms each, the fastest counts
    for (int repeat = -1; repeat < 3; repeat++) {
        CHECK(hipEventRecord(start));
        issue<CASE><<<cus, 256 * waves_per_simd>>>(out, clocks, updates, 1.0f);
        CHECK(hipEventRecord(stop));
        CHECK(hipEventSynchronize(stop));
        float ms = 0.0f;
        CHECK(hipEventElapsedTime(&ms, start, stop));
        if (repeat < 0) {
            if (ms < min_ms) updates = (int)(updates * (min_ms / ms) * 1.05) + 1;
            continue;
        }
        if (ms < best) {
            best = ms;
            CHECK(hipMemcpy(best_clocks, clocks, sizeof best_clocks, hipMemcpyDeviceToHost));
        }
    }
    const double instructions_per_simd = (double)waves_per_simd * updates * 64 * per_term[CASE];
    const double ns_per_instruction = best * 1e6 / instructions_per_simd;
    const double lane_ops_per_s = 1024.0 * 64.0 / (ns_per_instruction * 1e-9);
    const double mhz = (double)best_clocks[1] / ((double)best_clocks[0] / 100.0);
    const double terms = 30000.0 * 30000.0 * 1024.0;
    results[CASE][waves_per_simd] = {best, ns_per_instruction, lane_ops_per_s, mhz};
    printf("%-42s waves/SIMD %d  %8.3f ms  %.4f ns per wave instruction per SIMD  %6.2f T lane-ops/s  clock %4.0f MHz  %.3f cycles",
           case_names[CASE], waves_per_simd, best, ns_per_instruction, lane_ops_per_s / 1e12, mhz, ns_per_instruction * mhz * 1e-3);
    if (CASE <= POW_ROWS || CASE == SAD_U32)
        printf("  -> M = N = 30000, K = 1024 in %.1f ms", terms * per_term[CASE] / lane_ops_per_s * 1e3);
    printf("\n");
    fflush(stdout);
    return 0;
}

int main(int argc, char **argv)
{
    if (argc > 1 && !strcmp(argv[1], "walk")) return walk_ablations();
    const double min_ms = argc > 1 ? atof(argv[1]) : 3.0;
    float *out;
    long long *clocks;
    CHECK(hipMalloc(&out, 256 * 1024 * sizeof(float)));
    CHECK(hipMalloc(&clocks, 2 * sizeof(long long)));
    printf("every launch at least %.1f ms\n", min_ms);
    for (int waves = 2; waves <= 4; waves++) {
        if (measure<P1_ROWS>(out, clocks, waves, min_ms) || measure<P2_ROWS>(out, clocks, waves, min_ms) ||
            measure<POW_ROWS>(out, clocks, waves, min_ms) || measure<PLAIN_ADD>(out, clocks, waves, min_ms) ||
            measure<ABS_ADD>(out, clocks, waves, min_ms) || measure<EXP2>(out, clocks, waves, min_ms) ||
            measure<LOG2>(out, clocks, waves, min_ms) || measure<SAD_U32>(out, clocks, waves, min_ms))
            return 1;
    }
    // the cdist kernels hold 3 waves per SIMD (the fixed-point one 2); the best of 2 .. 4 is what the ALU can do
    printf("\nmin_launch_ms = %.1f\n", min_ms);
    for (int c = 0; c < CASES; c++) {
        int best = 2;
        for (int waves = 3; waves <= 4; waves++)
            if (results[c][waves].ns_per_instruction < results[c][best].ns_per_instruction) best = waves;
        const Result &r = results[c][best];
        printf("%s_lane_ops_per_s = %.4e\n%s_ns_per_instruction = %.4f\n%s_clock_mhz = %.0f\n%s_waves_per_simd = %d\n",
               case_keys[c], r.lane_ops_per_s, case_keys[c], r.ns_per_instruction, case_keys[c], r.mhz, case_keys[c], best);
    }
    CHECK(hipFree(out));
    CHECK(hipFree(clocks));
    return 0;
}
