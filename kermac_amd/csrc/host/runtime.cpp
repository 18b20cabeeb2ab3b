// Error reporting, device checks, and the hiprtc / hipModule wrappers of the C ABI.
#include "host_common.hpp"
#include "dispatch_rules.hpp"

#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace kmc_host {

static thread_local std::string g_last_error;

int fail(int code, const char *format, ...)
{
    char buffer[2048];
    va_list ap;
    va_start(ap, format);
    vsnprintf(buffer, sizeof buffer, format, ap);
    va_end(ap);
    g_last_error = buffer;
    return code;
}

int fail_hip(hipError_t error, const char *what)
{
    return fail(KMC_ERR_HIP_BASE + static_cast<int>(error), "%s: %s", what, hipGetErrorString(error));
}

void clear_error() { g_last_error.clear(); }

int require_gfx950()
{
    // One slot per device; 0 = unknown, 1 = gfx950, 2 = something else.
    static std::mutex mutex;
    static std::vector<int> verdict;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
    std::lock_guard<std::mutex> lock(mutex);
    if (device >= static_cast<int>(verdict.size())) verdict.resize(device + 1, 0);
    if (verdict[device] == 0) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, device);
        if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
        verdict[device] = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    }
    if (verdict[device] != 1) {
        return fail(KMC_ERR_WRONG_DEVICE, "device %d is not a gfx950 (MI355X); these kernels are built for gfx950 only", device);
    }
    return KMC_OK;
}

static int fail_rtc(hiprtcResult r, const char *what, const std::string &log)
{
    return fail(KMC_ERR_HIPRTC_BASE + static_cast<int>(r), "%s: %s\n%s", what, hiprtcGetErrorString(r), log.c_str());
}

}  // namespace kmc_host

using namespace kmc_host;

extern "C" {

int kmc_abi_version(void) { return KMC_ABI_VERSION; }

int kmc_dispatch_rules(char *buf, size_t buf_len)
{
    static const struct { const char *name; long long value; } rules[] = {
#define KMC_LIST_RULE(name, value) {#name, value},
        KMC_DISPATCH_RULES(KMC_LIST_RULE)
#undef KMC_LIST_RULE
    };
    if (!buf || buf_len == 0) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_dispatch_rules: no buffer");
    size_t used = 0;
    for (const auto &rule : rules) {
        const int wrote = std::snprintf(buf + used, buf_len - used, "%s = %lld\n", rule.name, rule.value);
        if (wrote < 0 || static_cast<size_t>(wrote) >= buf_len - used)
            return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_dispatch_rules: the buffer of %zu bytes is too small", buf_len);
        used += static_cast<size_t>(wrote);
    }
    return KMC_OK;
}

const char *kmc_last_error(void) { return g_last_error.c_str(); }

int kmc_device_arch(int device, char *buf, size_t buf_len)
{
    if (!buf || buf_len == 0) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_device_arch: no buffer");
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
    snprintf(buf, buf_len, "%s", prop.gcnArchName);
    return KMC_OK;
}

int kmc_jit_compile(const char *source, const char *source_name,
                    int n_headers, const char *const *headers, const char *const *header_names,
                    int n_options, const char *const *options,
                    int n_names, const char *const *name_expressions,
                    void **code, size_t *code_size, char **lowered_names)
{
    if (!source || !code || !code_size || n_headers < 0 || n_options < 0 || n_names < 0 ||
        (n_names > 0 && (!name_expressions || !lowered_names))) {
        return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_jit_compile: bad arguments");
    }
    *code = nullptr;
    *code_size = 0;
    hiprtcProgram program;
    hiprtcResult r = hiprtcCreateProgram(&program, source, source_name ? source_name : "kermac_amd_jit.hip",
                                         n_headers, const_cast<const char **>(headers),
                                         const_cast<const char **>(header_names));
    if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcCreateProgram", "");
    for (int i = 0; i < n_names; i++) {
        r = hiprtcAddNameExpression(program, name_expressions[i]);
        if (r != HIPRTC_SUCCESS) {
            hiprtcDestroyProgram(&program);
            return fail_rtc(r, "hiprtcAddNameExpression", name_expressions[i]);
        }
    }
    r = hiprtcCompileProgram(program, n_options, const_cast<const char **>(options));
    std::string log;
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(program, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        log.resize(log_size);
        hiprtcGetProgramLog(program, &log[0]);
    }
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&program);
        return fail_rtc(r, "hiprtcCompileProgram", log);
    }
    size_t size = 0;
    r = hiprtcGetCodeSize(program, &size);
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&program);
        return fail_rtc(r, "hiprtcGetCodeSize", log);
    }
    void *blob = malloc(size ? size : 1);
    r = hiprtcGetCode(program, static_cast<char *>(blob));
    if (r != HIPRTC_SUCCESS) {
        free(blob);
        hiprtcDestroyProgram(&program);
        return fail_rtc(r, "hiprtcGetCode", log);
    }
    for (int i = 0; i < n_names; i++) lowered_names[i] = nullptr;
    for (int i = 0; i < n_names; i++) {
        const char *lowered = nullptr;
        r = hiprtcGetLoweredName(program, name_expressions[i], &lowered);
        if (r != HIPRTC_SUCCESS || !lowered) {
            for (int j = 0; j < i; j++) { free(lowered_names[j]); lowered_names[j] = nullptr; }
            free(blob);
            hiprtcDestroyProgram(&program);
            return fail_rtc(r, "hiprtcGetLoweredName", name_expressions[i]);
        }
        lowered_names[i] = strdup(lowered);
    }
    hiprtcDestroyProgram(&program);
    *code = blob;
    *code_size = size;
    return KMC_OK;
}

void kmc_jit_free(void *ptr) { free(ptr); }

int kmc_module_load(const void *code, size_t code_size, void **module)
{
    if (!code || code_size == 0 || !module) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_module_load: bad arguments");
    int status = require_gfx950();
    if (status != KMC_OK) return status;
    hipModule_t handle = nullptr;
    hipError_t e = hipModuleLoadData(&handle, code);
    if (e != hipSuccess) return fail_hip(e, "hipModuleLoadData");
    *module = handle;
    return KMC_OK;
}

int kmc_module_get_function(void *module, const char *lowered_name, void **function)
{
    if (!module || !lowered_name || !function) return fail(KMC_ERR_INVALID_ARGUMENT, "kmc_module_get_function: bad arguments");
    hipFunction_t f = nullptr;
    hipError_t e = hipModuleGetFunction(&f, static_cast<hipModule_t>(module), lowered_name);
    if (e != hipSuccess) return fail_hip(e, lowered_name);
    *function = f;
    return KMC_OK;
}

int kmc_module_unload(void *module)
{
    if (!module) return KMC_OK;
    hipError_t e = hipModuleUnload(static_cast<hipModule_t>(module));
    if (e != hipSuccess) return fail_hip(e, "hipModuleUnload");
    return KMC_OK;
}

}  // extern "C"
