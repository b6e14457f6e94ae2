// Error state, version and device facts of the C ABI.
#include <cstring>
#include <map>
#include <mutex>

#include "host_common.h"
#include "host/ir.hpp"

namespace arkmi {

static thread_local std::string g_last_error;

void set_last_error(const std::string &msg) { g_last_error = msg; }

int current_device() {
    int dev = 0;
    ARKMI_HIP(hipGetDevice(&dev));
    return dev;
}

const DeviceFacts &device_facts(int device_id) {
    static std::mutex mu;
    static std::map<int, DeviceFacts> cache;
    std::lock_guard<std::mutex> lk(mu);
    auto it = cache.find(device_id);
    if (it != cache.end()) return it->second;
    hipDeviceProp_t prop;
    ARKMI_HIP(hipGetDeviceProperties(&prop, device_id));
    DeviceFacts f;
    f.num_cu = prop.multiProcessorCount;
    f.lds_bytes = (int)prop.maxSharedMemoryPerMultiProcessor;
    return cache.emplace(device_id, f).first->second;
}

}  // namespace arkmi

extern "C" {

const char *arkmi_last_error(void) { return arkmi::g_last_error.c_str(); }

const char *arkmi_version(void) { return "0.1.0"; }

int arkmi_init(void) {
    return arkmi::guard([&] { ark::reload_env(); });
}

int arkmi_device_info_get(int device_id, arkmi_device_info *out) {
    return arkmi::guard([&] {
        if (!out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "out is null");
        int n = 0;
        ARKMI_HIP(hipGetDeviceCount(&n));
        if (device_id < 0 || device_id >= n)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "invalid device id ", device_id, " (", n, " devices)");
        hipDeviceProp_t prop;
        ARKMI_HIP(hipGetDeviceProperties(&prop, device_id));
        std::memset(out, 0, sizeof(*out));
        out->device_id = device_id;
        out->num_cu = prop.multiProcessorCount;
        out->wave_size = prop.warpSize;
        out->max_threads_per_block = prop.maxThreadsPerBlock;
        out->lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
        out->l2_bytes = prop.l2CacheSize;
        out->hbm_bytes = prop.totalGlobalMem;
        out->clock_khz = prop.clockRate;
        std::strncpy(out->gcn_arch, prop.gcnArchName, sizeof(out->gcn_arch) - 1);
        // "gfx950:sramecc+:xnack-" -> "ROCM_950" (the reference builds the
        // name the same way, ark/gpu/gpu_manager.cpp:58-73).
        std::string g(prop.gcnArchName);
        size_t colon = g.find(':');
        if (colon != std::string::npos) g = g.substr(0, colon);
        std::string suffix = g.size() > 3 ? g.substr(3) : g;
        for (auto &c : suffix) c = (char)toupper((unsigned char)c);
        std::string arch = "ROCM_" + suffix;
        std::strncpy(out->arch, arch.c_str(), sizeof(out->arch) - 1);
    });
}

}  // extern "C"
