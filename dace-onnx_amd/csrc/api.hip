// Library identity, per-thread error channel and device query.
#include "common.h"

#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>

namespace mi355x {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* kernel_name) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return set_error(MI355X_ERR_LAUNCH, "%s: launch failed: %s", kernel_name, hipGetErrorString(e));
    return MI355X_OK;
}

// ---- launch parameters that do not change from call to call -------------------------------------
// The MI355X_* variables select kernel variants (used by the tests that run every tile shape) and the CU
// count sizes persistent grids. Both are looked up once: the environment on first use (again after
// mi355x_reload_tuning()), the CU count once per device.
static Tuning g_tuning;
static std::atomic<bool> g_tuning_valid{false};
static std::mutex g_tuning_mutex;

#ifdef MI355X_WG_TRACE
unsigned long long* trace_buffer(unsigned* capacity) {
    const char* v = getenv("MI355X_WG_TRACE_BUFFER");
    const char* c = getenv("MI355X_WG_TRACE_CAPACITY");
    *capacity = c && *c ? (unsigned)strtoul(c, nullptr, 10) : 0u;
    return v && *v && *capacity ? reinterpret_cast<unsigned long long*>(strtoull(v, nullptr, 10)) : nullptr;
}
#endif

static int env_int(const char* name, int fallback) {
    const char* v = getenv(name);
    return v && *v ? atoi(v) : fallback;
}

static void parse_tuning(Tuning& t) {
    const char* c = getenv("MI355X_GEMM_CONFIG");
    t.gemm_config = c && c[0] >= '0' && c[0] <= '9' ? c[0] - '0' : -1;
    t.gemm_nt_bn = env_int("MI355X_GEMM_NT_BN", 0);
    t.gemm_nt_bk = env_int("MI355X_GEMM_NT_BK", 0);
    t.gemm_nt_bm = env_int("MI355X_GEMM_NT_BM", 0);
    t.gemm_nt_per_cu = env_int("MI355X_GEMM_NT_PER_CU", 0);
    t.gemm_nt_waves = env_int("MI355X_GEMM_NT_WAVES", 0);
    t.gemm_group_m = env_int("MI355X_GEMM_GROUP_M", 0);
    t.gemm_ksplit = env_int("MI355X_GEMM_KSPLIT", -1);
    c = getenv("MI355X_CONV_CONFIG");
    t.conv_config = c && c[0] >= '0' && c[0] <= '9' ? c[0] - '0' : -1;
    t.conv_gather_bn = env_int("MI355X_CONV_GATHER_BN", 0);
    t.conv_tail = env_int("MI355X_CONV_TAIL", -1);
    t.conv_static_taps = env_int("MI355X_CONV_STATIC_TAPS", 1);
    t.conv_per_cu = env_int("MI355X_CONV_PER_CU", 0);
    t.mmi_generic = getenv("MI355X_MMI_GENERIC") != nullptr;
    t.mmi_wgs_per_cu = env_int("MI355X_MMI_WGS_PER_CU", 0);
    t.mmi_tile = env_int("MI355X_MMI_TILE", 0);
    t.attn_waves = env_int("MI355X_ATTN_WAVES", 0);
}

Tuning tuning() {
    // every read of the struct happens under the lock mi355x_reload_tuning() writes it under; a launch works on its copy
    std::lock_guard<std::mutex> lock(g_tuning_mutex);
    if (!g_tuning_valid.load(std::memory_order_relaxed)) {
        parse_tuning(g_tuning);
        g_tuning_valid.store(true, std::memory_order_relaxed);
    }
    return g_tuning;
}

int device_cus() {
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> cached[MAX_DEVICES];   // 0: not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (dev < 0 || dev >= MAX_DEVICES) return mi355x_device_cu_count();
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        cus = mi355x_device_cu_count();
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

__global__ void empty_kernel() {}

}  // namespace mi355x

extern "C" {

int mi355x_launch_empty_kernel(void* stream) {
    hipLaunchKernelGGL(mi355x::empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream));
    return mi355x::check_launch("empty_kernel");
}

void mi355x_reload_tuning(void) {
    std::lock_guard<std::mutex> lock(mi355x::g_tuning_mutex);
    mi355x::parse_tuning(mi355x::g_tuning);
    mi355x::g_tuning_valid.store(true, std::memory_order_release);
}

int mi355x_version(void) { return MI355X_ONNX_VERSION; }

const char* mi355x_last_error(void) { return mi355x::g_last_error; }

int mi355x_device_cu_count(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return cus;
}

}  // extern "C"
