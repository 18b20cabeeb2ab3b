// What one MI355X issues for the instruction mixes of the three cdist inner loops, with
// nothing but registers involved: the rank-1 updates of kmc::build_kernel
// (csrc/kernels/build_kernel.hpp: row_abs_diff for p = 1, row_square_diff for p = 2,
// row_pow_diff for a fractional p) run on fragments that never change, no LDS, no memory.
// The rates printed here are the issue ceilings that the cdist kernels are measured
// against (bench.py: frac_of_issue_ceiling): a kernel cannot retire its 2 (p = 1, 2) or 5
// (fractional p, two of them transcendental) instructions per (m, n, k) faster than this.
//
//   kermac_amd/_lib/valu_issue_rates            (built by `python -m kermac_amd._build`)
//
// Per case and per number of waves on a SIMD: time, nanoseconds per wave instruction per
// SIMD, lane operations per second for the whole chip, the shader clock during the run
// (clock64 ticks per microsecond of the 100 MHz wall clock), and the time the M = N = 30000,
// K = 1024 problem would take at that rate.
#include <hip/hip_runtime.h>

#include <cstdio>

#include "../kermac_amd/csrc/kernels/build_kernel.hpp"

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
// vector instructions per (m, n, k) of the case, and per 8 x 8 rank-1 update
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

template <int CASE>
int measure(float *out, long long *clocks, int waves_per_simd)
{
    // one workgroup of 4 * waves_per_simd waves on every CU: each SIMD holds waves_per_simd of them
    const int cus = 256, updates = (CASE == POW_ROWS || CASE == EXP2 || CASE == LOG2) ? 1500 : 6000;
    hipEvent_t start, stop;
    CHECK(hipEventCreate(&start));
    CHECK(hipEventCreate(&stop));
    issue<CASE><<<cus, 256 * waves_per_simd>>>(out, clocks, 10, 1.0f);
    CHECK(hipDeviceSynchronize());
    float best = 1e30f;
    long long best_clocks[2] = {1, 0};
    for (int repeat = 0; repeat < 3; repeat++) {
        CHECK(hipEventRecord(start));
        issue<CASE><<<cus, 256 * waves_per_simd>>>(out, clocks, updates, 1.0f);
        CHECK(hipEventRecord(stop));
        CHECK(hipEventSynchronize(stop));
        float ms = 0.0f;
        CHECK(hipEventElapsedTime(&ms, start, stop));
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
    printf("%-42s waves/SIMD %d  %7.3f ms  %.4f ns per wave instruction per SIMD  %6.2f T lane-ops/s  clock %4.0f MHz",
           case_names[CASE], waves_per_simd, best, ns_per_instruction, lane_ops_per_s / 1e12, mhz);
    if (CASE <= POW_ROWS)
        printf("  -> M = N = 30000, K = 1024 in %.1f ms", terms * per_term[CASE] / lane_ops_per_s * 1e3);
    printf("\n");
    return 0;
}

int main()
{
    float *out;
    long long *clocks;
    CHECK(hipMalloc(&out, 256 * 1024 * sizeof(float)));
    CHECK(hipMalloc(&clocks, 2 * sizeof(long long)));
    for (int waves = 2; waves <= 4; waves++) {
        if (measure<P1_ROWS>(out, clocks, waves) || measure<P2_ROWS>(out, clocks, waves) ||
            measure<POW_ROWS>(out, clocks, waves) || measure<PLAIN_ADD>(out, clocks, waves) ||
            measure<ABS_ADD>(out, clocks, waves) || measure<EXP2>(out, clocks, waves) || measure<LOG2>(out, clocks, waves) ||
            measure<SAD_U32>(out, clocks, waves))
            return 1;
    }
    CHECK(hipFree(out));
    CHECK(hipFree(clocks));
    return 0;
}
