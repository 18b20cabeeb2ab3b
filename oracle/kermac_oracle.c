/*
 * CPU oracle for the fused distance hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference's two
 * production kernels.  It exists to check the HIP kernels; it is never part of
 * the product path.  Only tests, the smoke check and the benchmark's CPU
 * baseline leg may build or call it.
 *
 * Every routine has two modes selected by `wide`:
 *   wide = 1  all arithmetic in double: the "truth" the GPU results are
 *             compared against with a relative tolerance;
 *   wide = 0  fp32 arithmetic in the reference's operation order (fp32
 *             subtract, fp32 power, fp32 sequential accumulate).
 *
 * Reference semantics followed (file:line under the reference checkout):
 *   include/build_a_kernel.cuh:339-370   inner operator + inner power + accumulate
 *   include/build_a_kernel.cuh:374-392   outer power
 *   include/build_a_kernel.cuh:394-404   epsilon mask (kernel_type != NONE)
 *   include/build_a_kernel.cuh:406-427   Laplace / Gaussian kernel function
 *   include/build_a_kernel.cuh:429-447   diagonal regularisation
 *   include/p_norm_gradient.cuh:100-104, 373-394   gradient inner loop
 *   include/kermac_internal_common.cuh:76-192      _abs/_sqrt/_exp/_pow/_signum
 *
 * Parity pins (tests/test_oracle.py): torch.cdist in fp64 for the p-norm
 * descriptors, numpy brute force on tiny inputs, closed forms (identical
 * points, zero operand, K = 1), numpy compositions for the kernel functions,
 * the reference test's einsum identity for the p = 2 gradient and an
 * independent numpy brute force for the p = 1 / fractional-p gradient.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>

enum { KMO_OP_DIFF = 0, KMO_OP_DOT = 1 };
enum { KMO_POW_NOOP = 0, KMO_POW_ABS = 1, KMO_POW_SQUARE = 2, KMO_POW_SQRT = 3, KMO_POW_POW = 4 };
enum { KMO_KERNEL_NONE = 0, KMO_KERNEL_LAPLACE = 1, KMO_KERNEL_GAUSSIAN = 2 };
enum { KMO_NORM_L1 = 0, KMO_NORM_L2 = 1, KMO_NORM_P = 2 };

/* _pow(v, p) = ex2(p * lg2(v)): include/kermac_internal_common.cuh:139-161.
 * pow(0, p>0) = 0, pow(0, 0) = NaN (0 * -inf), negative v gives NaN. */
static double pow_via_log2_d(double v, double p) { return exp2(p * log2(v)); }
static float pow_via_log2_f(float v, float p) { return exp2f(p * log2f(v)); }

static double apply_power_d(int kind, double v, double p)
{
    switch (kind) {
    case KMO_POW_NOOP: return v;
    case KMO_POW_ABS: return fabs(v);
    case KMO_POW_SQUARE: return v * v;
    case KMO_POW_SQRT: return sqrt(v);
    case KMO_POW_POW: return pow_via_log2_d(v, p);
    default: return NAN;
    }
}

static float apply_power_f(int kind, float v, float p)
{
    switch (kind) {
    case KMO_POW_NOOP: return v;
    case KMO_POW_ABS: return fabsf(v);
    case KMO_POW_SQUARE: return v * v;
    case KMO_POW_SQRT: return sqrtf(v);
    case KMO_POW_POW: return pow_via_log2_f(v, p);
    default: return NAN;
    }
}

/*
 * out view C[l, m, n] = kernel_fn(outer(sum_k inner(B[l,n,k] (-|*) A[l,m,k])))
 * All strides are in elements; a batch stride of 0 broadcasts.
 * Hyper-parameter arrays are indexed [l * stride] (stride 0 = shared scalar).
 */
void kmo_build_kernel(
    int inner_operator, int inner_power, int outer_power, int kernel_type,
    int M, int N, int K, int L,
    const float *A, int64_t a_sm, int64_t a_sk, int64_t a_sl,
    const float *B, int64_t b_sn, int64_t b_sk, int64_t b_sl,
    float *C, int64_t c_sm, int64_t c_sn, int64_t c_sl,
    const float *p_inner, int64_t p_inner_sl,
    const float *p_outer, int64_t p_outer_sl,
    const float *bandwidth, int64_t bandwidth_sl,
    const float *regularization, int64_t regularization_sl,
    int regularization_offset_x, int regularization_offset_y,
    float epsilon, int wide)
{
    for (int l = 0; l < L; l++) {
        const float ppi = p_inner ? p_inner[l * p_inner_sl] : 0.0f;
        const float ppo = p_outer ? p_outer[l * p_outer_sl] : 0.0f;
        const float bw = bandwidth ? bandwidth[l * bandwidth_sl] : 0.0f;
        const float reg = regularization ? regularization[l * regularization_sl] : 0.0f;
#pragma omp parallel for schedule(static)
        for (int m = 0; m < M; m++) {
            const float *a_row = A + l * a_sl + (int64_t)m * a_sm;
            for (int n = 0; n < N; n++) {
                const float *b_row = B + l * b_sl + (int64_t)n * b_sn;
                double result;
                if (wide) {
                    double acc = 0.0;
                    for (int k = 0; k < K; k++) {
                        double av = a_row[k * a_sk], bv = b_row[k * b_sk];
                        double t = inner_operator == KMO_OP_DIFF ? bv - av : bv * av;
                        if (inner_power == KMO_POW_POW) t = fabs(t); /* build_a_kernel.cuh:361-363 */
                        acc += apply_power_d(inner_power, t, (double)ppi);
                    }
                    acc = apply_power_d(outer_power, acc, (double)ppo);
                    if (kernel_type != KMO_KERNEL_NONE && acc < (double)epsilon) acc = 0.0;
                    if (kernel_type == KMO_KERNEL_LAPLACE) {
                        acc = exp(-acc / (double)bw);
                    } else if (kernel_type == KMO_KERNEL_GAUSSIAN) {
                        acc = exp(-acc / (2.0 * (double)bw * (double)bw));
                    }
                    result = acc;
                } else {
                    float acc = 0.0f;
                    for (int k = 0; k < K; k++) {
                        float av = a_row[k * a_sk], bv = b_row[k * b_sk];
                        float t = inner_operator == KMO_OP_DIFF ? bv - av : bv * av;
                        if (inner_power == KMO_POW_POW) t = fabsf(t);
                        acc += apply_power_f(inner_power, t, ppi);
                    }
                    acc = apply_power_f(outer_power, acc, ppo);
                    if (kernel_type != KMO_KERNEL_NONE && acc < epsilon) acc = 0.0f;
                    if (kernel_type == KMO_KERNEL_LAPLACE) {
                        float gamma = 1.0f / bw;
                        acc = expf(acc * -gamma);
                    } else if (kernel_type == KMO_KERNEL_GAUSSIAN) {
                        float gamma = 1.0f / (2 * bw * bw);
                        acc = expf(acc * -gamma);
                    }
                    result = acc;
                }
                /* build_a_kernel.cuh:429-447: the value is REPLACED by 1 + reg. */
                if (kernel_type != KMO_KERNEL_NONE && reg != 0.0f &&
                    regularization_offset_x + m == regularization_offset_y + n) {
                    result = wide ? 1.0 + (double)reg : (double)(float)(1.0 + reg);
                }
                C[l * c_sl + (int64_t)m * c_sm + (int64_t)n * c_sn] = (float)result;
            }
        }
    }
}

/*
 * E[l, o, n, m] = sum_k C[l,o,k] * A[l,k,m] * g(D[l,n,m] - B[l,n,k])
 *   g = copysign(1, x)                 (L1)
 *   g = x                              (L2; no factor 2)
 *   g = copysign(1, x) * |x|^(p - 1)   (P)
 * copysign, not sign(): g(+0) = +1, g(-0) = -1
 * (include/kermac_internal_common.cuh:178-192).
 */
void kmo_norm_kernel_gradient(
    int norm_type,
    int M, int N, int O, int K, int L,
    const float *A, int64_t a_sk, int64_t a_sm, int64_t a_sl,
    const float *B, int64_t b_sn, int64_t b_sk, int64_t b_sl,
    const float *Cc, int64_t c_so, int64_t c_sk, int64_t c_sl,
    const float *D, int64_t d_sn, int64_t d_sm, int64_t d_sl,
    float *E, int64_t e_so, int64_t e_sn, int64_t e_sm, int64_t e_sl,
    const float *P, int64_t p_sl, int wide)
{
    for (int l = 0; l < L; l++) {
        const float p_minus_1 = norm_type == KMO_NORM_P ? P[l * p_sl] - 1.0f : 0.0f;
#pragma omp parallel for schedule(static) collapse(2)
        for (int n = 0; n < N; n++) {
            for (int m = 0; m < M; m++) {
                const float dv = D[l * d_sl + (int64_t)n * d_sn + (int64_t)m * d_sm];
                double acc_d[O];
                float acc_f[O];
                for (int o = 0; o < O; o++) { acc_d[o] = 0.0; acc_f[o] = 0.0f; }
                for (int k = 0; k < K; k++) {
                    const float av = A[l * a_sl + (int64_t)k * a_sk + (int64_t)m * a_sm];
                    const float bv = B[l * b_sl + (int64_t)n * b_sn + (int64_t)k * b_sk];
                    const float *c_col = Cc + l * c_sl + (int64_t)k * c_sk;
                    if (wide) {
                        double diff = (double)dv - (double)bv;
                        double sign = copysign(1.0, diff);
                        double g;
                        if (norm_type == KMO_NORM_L1) g = sign;
                        else if (norm_type == KMO_NORM_L2) g = diff;
                        else g = pow_via_log2_d(fabs(diff), (double)p_minus_1) * sign;
                        g = (double)av * g;
                        for (int o = 0; o < O; o++) acc_d[o] += (double)c_col[(int64_t)o * c_so] * g;
                    } else {
                        float diff = dv - bv;
                        float sign = copysignf(1.0f, diff);
                        float g;
                        if (norm_type == KMO_NORM_L1) g = sign;
                        else if (norm_type == KMO_NORM_L2) g = diff;
                        else g = pow_via_log2_f(fabsf(diff), p_minus_1) * sign;
                        g = av * g;
                        for (int o = 0; o < O; o++) acc_f[o] += c_col[(int64_t)o * c_so] * g;
                    }
                }
                for (int o = 0; o < O; o++) {
                    E[l * e_sl + (int64_t)o * e_so + (int64_t)n * e_sn + (int64_t)m * e_sm] =
                        wide ? (float)acc_d[o] : acc_f[o];
                }
            }
        }
    }
}

/*
 * Fused kernel-matrix x coefficients (no counterpart kernel in the reference;
 * defined as the composition run_kernel(descriptor, a, b, ...) @ coefficients):
 *   out[l, m, o] = sum_n kernelvalue[l, m, n] * coef[l, n, o]
 * with kernelvalue exactly as kmo_build_kernel computes it.
 */
void kmo_kernel_times_coefficients(
    int inner_operator, int inner_power, int outer_power, int kernel_type,
    int M, int N, int K, int O, int L,
    const float *A, int64_t a_sm, int64_t a_sk, int64_t a_sl,
    const float *B, int64_t b_sn, int64_t b_sk, int64_t b_sl,
    const float *coef, int64_t w_sn, int64_t w_so, int64_t w_sl,
    float *out, int64_t o_sm, int64_t o_so, int64_t o_sl,
    const float *p_inner, int64_t p_inner_sl,
    const float *p_outer, int64_t p_outer_sl,
    const float *bandwidth, int64_t bandwidth_sl,
    const float *regularization, int64_t regularization_sl,
    int regularization_offset_x, int regularization_offset_y,
    float epsilon, int wide)
{
    for (int l = 0; l < L; l++) {
        const float ppi = p_inner ? p_inner[l * p_inner_sl] : 0.0f;
        const float ppo = p_outer ? p_outer[l * p_outer_sl] : 0.0f;
        const float bw = bandwidth ? bandwidth[l * bandwidth_sl] : 0.0f;
        const float reg = regularization ? regularization[l * regularization_sl] : 0.0f;
#pragma omp parallel for schedule(static)
        for (int m = 0; m < M; m++) {
            const float *a_row = A + l * a_sl + (int64_t)m * a_sm;
            double acc_o[256];
            for (int o = 0; o < O && o < 256; o++) acc_o[o] = 0.0;
            for (int n = 0; n < N; n++) {
                const float *b_row = B + l * b_sl + (int64_t)n * b_sn;
                double acc = 0.0;
                float accf = 0.0f;
                for (int k = 0; k < K; k++) {
                    if (wide) {
                        double av = a_row[k * a_sk], bv = b_row[k * b_sk];
                        double t = inner_operator == KMO_OP_DIFF ? bv - av : bv * av;
                        if (inner_power == KMO_POW_POW) t = fabs(t);
                        acc += apply_power_d(inner_power, t, (double)ppi);
                    } else {
                        float av = a_row[k * a_sk], bv = b_row[k * b_sk];
                        float t = inner_operator == KMO_OP_DIFF ? bv - av : bv * av;
                        if (inner_power == KMO_POW_POW) t = fabsf(t);
                        accf += apply_power_f(inner_power, t, ppi);
                    }
                }
                if (wide) {
                    acc = apply_power_d(outer_power, acc, (double)ppo);
                    if (kernel_type != KMO_KERNEL_NONE && acc < (double)epsilon) acc = 0.0;
                    if (kernel_type == KMO_KERNEL_LAPLACE) acc = exp(-acc / (double)bw);
                    else if (kernel_type == KMO_KERNEL_GAUSSIAN) acc = exp(-acc / (2.0 * (double)bw * (double)bw));
                } else {
                    accf = apply_power_f(outer_power, accf, ppo);
                    if (kernel_type != KMO_KERNEL_NONE && accf < epsilon) accf = 0.0f;
                    if (kernel_type == KMO_KERNEL_LAPLACE) accf = expf(accf * -(1.0f / bw));
                    else if (kernel_type == KMO_KERNEL_GAUSSIAN) accf = expf(accf * -(1.0f / (2 * bw * bw)));
                    acc = accf;
                }
                if (kernel_type != KMO_KERNEL_NONE && reg != 0.0f &&
                    regularization_offset_x + m == regularization_offset_y + n) {
                    acc = 1.0 + (double)reg;
                }
                for (int o = 0; o < O && o < 256; o++) {
                    acc_o[o] += acc * (double)coef[l * w_sl + (int64_t)n * w_sn + (int64_t)o * w_so];
                }
            }
            for (int o = 0; o < O && o < 256; o++) {
                out[l * o_sl + (int64_t)m * o_sm + (int64_t)o * o_so] = (float)acc_o[o];
            }
        }
    }
}

int kmo_abi_version(void) { return 1; }
