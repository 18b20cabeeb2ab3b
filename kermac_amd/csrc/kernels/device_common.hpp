// Shared device-side definitions for the gfx950 kernels.
//
// This header is compiled two ways: ahead of time by hipcc into the C-ABI
// library, and at run time by hiprtc for descriptor variants outside the
// ahead-of-time set.  It therefore includes nothing from the host C++ library
// and uses only builtin types.
//
// Enumerator values are part of the C ABI (see kermac_amd.h) and of the
// on-disk kernel cache key; never renumber them.
#pragma once

namespace kmc {

// Reference enums: include/kermac_internal_common.cuh:41-74.
enum InnerOperator : int { OP_DIFF = 0, OP_DOT = 1 };
enum PowerType : int { POW_NOOP = 0, POW_ABS = 1, POW_SQUARE = 2, POW_SQRT = 3, POW_POW = 4 };
// Not part of the C ABI: inner powers the host substitutes for POW_POW when the
// exponent is a scalar equal to 0.5, 1.5, 3 or 4.  |x|^p then needs one square
// root or none instead of a logarithm and an exponential.
enum SpecialPower : int { POW_ABS_HALF = 5, POW_ABS_THREE_HALVES = 6, POW_ABS_CUBE = 7, POW_ABS_FOURTH = 8 };
enum KernelType : int { KERNEL_NONE = 0, KERNEL_LAPLACE = 1, KERNEL_GAUSSIAN = 2 };
enum NormType : int { NORM_L1 = 0, NORM_L2 = 1, NORM_P = 2 };

// How one operand panel (rows x K) is fetched from HBM.
//   COL: the row index (m or n) is the contiguous one ("K-major panel" a[K,M]).
//   ROW: k is the contiguous one (torch's default a[M,K]).
//   VEC: base pointer, leading dimension and batch stride are all multiples of
//        16 bytes, so 128-bit loads are legal.
enum LoadMode : int { LOAD_COL_VEC = 0, LOAD_COL_SCALAR = 1, LOAD_ROW_VEC = 2, LOAD_ROW_SCALAR = 3 };

typedef long long i64;

// Hardware transcendental: v_log_f32 / v_exp_f32 are base-2 and ~1 ulp.
// |x|^p as exp2(p * log2|x|), the reference's _pow (kermac_internal_common.cuh:139-161):
// gives 0 for x = 0, p > 0 and NaN for x = 0, p = 0.
__device__ __forceinline__ float fast_pow_abs(float x_abs, float p)
{
    return __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(x_abs));
}

// copysign(1, v): +1 for +0, -1 for -0 (kermac_internal_common.cuh:178-192).
__device__ __forceinline__ float signum(float v)
{
    return __builtin_copysignf(1.0f, v);
}

// `diff_sign` is -1 when the host swapped the operands (row-major result) and
// +1 otherwise; only the sign-sensitive inner powers look at it.
template <int INNER_OP, int INNER_POW>
__device__ __forceinline__ float inner_term(float a, float b, float p_inner, float diff_sign)
{
    // include/build_a_kernel.cuh:343-366
    float t = INNER_OP == OP_DIFF ? b - a : b * a;
    if (INNER_OP == OP_DIFF && (INNER_POW == POW_NOOP || INNER_POW == POW_SQRT)) t *= diff_sign;
    if (INNER_POW == POW_NOOP) return t;
    if (INNER_POW == POW_ABS) return __builtin_fabsf(t);
    if (INNER_POW == POW_SQUARE) return t * t;
    if (INNER_POW == POW_SQRT) return __builtin_amdgcn_sqrtf(t);
    const float x = __builtin_fabsf(t);
    if (INNER_POW == POW_ABS_HALF) return __builtin_amdgcn_sqrtf(x);
    if (INNER_POW == POW_ABS_THREE_HALVES) return x * __builtin_amdgcn_sqrtf(x);
    if (INNER_POW == POW_ABS_CUBE) return x * (t * t);
    if (INNER_POW == POW_ABS_FOURTH) return (t * t) * (t * t);
    return fast_pow_abs(x, p_inner);
}

// Epilogue of one accumulator: outer power, epsilon mask, kernel function.
// include/build_a_kernel.cuh:374-427.  Runs once per output element, so the
// accurate library routines are used for the exponentials and logarithms.  The
// square root is the hardware instruction (1 ulp, like the reference's
// sqrt.approx): the library routine's refinement costs 0.55 ms per 9e8 outputs,
// more than half the run time of a store-bound (small K) Euclidean distance.
__device__ __forceinline__ float epilogue_value(
    float acc, int outer_power, int kernel_type, float p_outer, float neg_gamma, float epsilon)
{
    switch (outer_power) {
    case POW_ABS: acc = __builtin_fabsf(acc); break;
    case POW_SQUARE: acc = acc * acc; break;
    case POW_SQRT: acc = __builtin_amdgcn_sqrtf(acc); break;
    case POW_POW: acc = exp2f(p_outer * log2f(acc)); break;
    default: break;
    }
    if (kernel_type != KERNEL_NONE) {
        if (acc < epsilon) acc = 0.0f;
        acc = expf(acc * neg_gamma);
    }
    return acc;
}

// -1/bandwidth (Laplace) or -1/(2 bandwidth^2) (Gaussian).
__device__ __forceinline__ float kernel_neg_gamma(int kernel_type, float bandwidth)
{
    if (kernel_type == KERNEL_LAPLACE) return -(1.0f / bandwidth);
    if (kernel_type == KERNEL_GAUSSIAN) return -(1.0f / (2.0f * bandwidth * bandwidth));
    return 0.0f;
}

// 4 consecutive floats starting at p; elements at index >= valid read as 0.
// `vec` says that p is 16-byte aligned.
__device__ __forceinline__ float4 load4_guarded(const float *p, int valid, bool vec)
{
    if (vec && valid >= 4) return *reinterpret_cast<const float4 *>(p);
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (valid > 0) v.x = p[0];
    if (valid > 1) v.y = p[1];
    if (valid > 2) v.z = p[2];
    if (valid > 3) v.w = p[3];
    return v;
}

}  // namespace kmc
