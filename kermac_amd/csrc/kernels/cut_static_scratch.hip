// kmc_build_kernel_cut_static: the contraction cut over k (kmc_build_kernel on ranges of
// k, then kmc_build_kernel_finish) as ONE entry point that allocates nothing, for callers
// that cannot call hipMalloc: code under HIP graph capture, tight serving loops, harnesses
// that forbid allocation.  The partial sums, which the two-call form keeps in a buffer the
// caller brings, live in a static device array of this library.
//
// That array exists once per GPU (each device that loads the library's code object holds
// its own copy, at its own address, until the process ends).  Its name is a host-side
// stand-in, not a device address: host code obtains the address with hipGetSymbolAddress,
// once per device with that device current, and uses only that pointer afterwards.  All
// calls on one GPU share the array, so two calls that overlap on one GPU (different
// streams, different host threads) race on it; calls on one stream are ordered.
// The first call on a device looks the address up (a lock, hipGetSymbolAddress, possibly the
// load of the code object): make one eager call per device before capturing calls into a graph.
#include <hip/hip_runtime.h>

#include <mutex>
#include <vector>

#include "../host/host_common.hpp"

namespace {

constexpr size_t SCRATCH_FLOATS = KMC_STATIC_SCRATCH_BYTES / sizeof(float);

// Partial sums (range, n, m) of the call in flight.  Every element that the finishing
// kernel reads has been written by the ranges launch of the same call, so nothing has
// to start at zero and the contents left by an earlier call are never seen.
__device__ __align__(256) float scratch[SCRATCH_FLOATS];

// Address of `scratch` on each device, looked up on the first call there.
int scratch_on_current_device(float **address)
{
    static std::mutex mutex;
    static std::vector<float *> per_device;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return kmc_host::fail_hip(e, "hipGetDevice");
    std::lock_guard<std::mutex> lock(mutex);
    if (device >= static_cast<int>(per_device.size())) per_device.resize(device + 1, nullptr);
    if (!per_device[device]) {
        float *ptr = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return kmc_host::fail_hip(e, "hipGetSymbolAddress(scratch)");
        if (!ptr) return kmc_host::fail(KMC_ERR_INVALID_ARGUMENT, "hipGetSymbolAddress returned a null address for the scratch array");
        per_device[device] = ptr;
    }
    *address = per_device[device];
    return KMC_OK;
}

}  // namespace

extern "C" int kmc_build_kernel_cut_static(const kmc_build_kernel_params *params, int32_t ranges, void *stream)
{
    using kmc_host::fail;
    if (!params) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    if (params->l != 1) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_build_kernel_cut_static takes one problem (l = 1), got l = %d", params->l);
    if (params->k_total != 0) return fail(KMC_ERR_INVALID_ARGUMENT, "k_total must be 0: the ranges are made here");
    if (params->flags & (KMC_FLAG_L2_GRAM | KMC_FLAG_L2_GRAM_BF16 | KMC_FLAG_DOT_PIECES | KMC_FLAG_L1_FIXED))
        return fail(KMC_ERR_INVALID_ARGUMENT, "the matrix-core and fixed-point flags cannot be combined with a cut over k");
    if (ranges < 1) return fail(KMC_ERR_INVALID_ARGUMENT, "ranges = %d, need at least 1", ranges);
    if (params->m < 0 || params->n < 0 || params->k < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative extent (m=%d n=%d k=%d)", params->m, params->n, params->k);
    if (!kmc_build_kernel_has_variant(params->inner_operator, params->inner_power))
        return fail(KMC_ERR_UNSUPPORTED_VARIANT, "inner_operator=%d inner_power=%d is not compiled ahead of time",
                    params->inner_operator, params->inner_power);

    // What the finishing call would reject is rejected here, before the ranges are launched.
    if (params->m > 0 && params->n > 0 && !params->c) return fail(KMC_ERR_INVALID_ARGUMENT, "c: null pointer");
    if (params->n > 1 && params->c_ld < params->m)
        return fail(KMC_ERR_INVALID_ARGUMENT, "c: leading dimension %lld is smaller than m=%d",
                    static_cast<long long>(params->c_ld), params->m);
    if (params->c_ld < 0 || params->c_bs < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "c: negative stride");
    // The array belongs to the current device, and so must the stream.
    if (stream) {
        int current = 0, of_stream = 0;
        hipError_t e = hipGetDevice(&current);
        if (e == hipSuccess) e = hipStreamGetDevice(static_cast<hipStream_t>(stream), &of_stream);
        if (e != hipSuccess) return kmc_host::fail_hip(e, "hipStreamGetDevice");
        if (current != of_stream)
            return fail(KMC_ERR_INVALID_ARGUMENT, "the stream belongs to device %d, the current device is %d", of_stream, current);
    }

    // Ranges of whole 16-term slices; the last one takes what is left of k.
    const int64_t k = params->k;
    int64_t depth = (k + ranges - 1) / ranges;
    depth = (depth + 15) / 16 * 16;
    if (depth < 16) depth = 16;
    const int64_t used = k > 0 ? (k + depth - 1) / depth : 1;
    const int64_t ld = (static_cast<int64_t>(params->m) + 3) / 4 * 4;      // 16-byte rows: 128-bit access
    const int64_t plane = ld * params->n;
    if (static_cast<double>(plane) * static_cast<double>(used) > static_cast<double>(SCRATCH_FLOATS))
        return fail(KMC_ERR_INVALID_ARGUMENT,
                    "%lld ranges of a %d x %d result need %.1f MiB of partial sums; the static array holds %d MiB "
                    "(use fewer ranges, or kmc_build_kernel + kmc_build_kernel_finish with a buffer of your own)",
                    static_cast<long long>(used), params->m, params->n,
                    static_cast<double>(plane) * static_cast<double>(used) * 4.0 / (1 << 20),
                    static_cast<int>(KMC_STATIC_SCRATCH_BYTES >> 20));

    float *partials = nullptr;
    int status = scratch_on_current_device(&partials);
    if (status != KMC_OK) return status;

    kmc_build_kernel_params sums = *params;
    sums.outer_power = KMC_POW_NOOP;
    sums.kernel_type = KMC_KERNEL_NONE;
    sums.k = static_cast<int32_t>(k > 0 ? depth : 0);
    sums.l = static_cast<int32_t>(used);
    sums.k_total = static_cast<int32_t>(k);         // 0 when k = 0: one "range" of no terms stores zeros
    sums.a_bs = depth * (params->a_majorness == KMC_COL_MAJOR ? params->a_ld : 1);
    sums.b_bs = depth * (params->b_majorness == KMC_COL_MAJOR ? params->b_ld : 1);
    sums.c = partials;
    sums.c_ld = ld;
    sums.c_bs = plane;
    status = kmc_build_kernel(&sums, stream);
    if (status != KMC_OK) return status;
    return kmc_build_kernel_finish(params, partials, ld, 0, plane, static_cast<int32_t>(used), stream);
}
