// Process-level pieces of the C ABI: device binding, the error string, the tuning table.

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "btb_common.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

int32_t attn_static_bind();  // glue.hip: resolves the static attention scratch on the current device

static DeviceInfo g_dev;
static std::mutex g_dev_lock;
static thread_local char g_err[256] = "";

void set_error(const char* msg) {
    std::snprintf(g_err, sizeof(g_err), "%s", msg);
}

int32_t hip_status(hipError_t e, const char* what) {
    if (e == hipSuccess) return OK;
    std::snprintf(g_err, sizeof(g_err), "[hip] %s failed: %d %s", what, (int)e, hipGetErrorString(e));
    return ERR_PANIC;
}

static int32_t bind_current() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDeviceProperties");
    g_dev.cus = prop.multiProcessorCount;
    g_dev.lds_bytes = (int)prop.maxSharedMemoryPerMultiProcessor;
    if (g_dev.lds_bytes <= 0) g_dev.lds_bytes = (int)prop.sharedMemPerBlock;
    g_dev.ready = true;
    return OK;
}

const DeviceInfo& device_info() {
    if (!g_dev.ready) {
        std::lock_guard<std::mutex> hold(g_dev_lock);
        if (!g_dev.ready && bind_current() != OK) {
            // a device that cannot be read: the launch that follows reports the failure itself
            g_dev.cus = 256;
            g_dev.lds_bytes = 64 * 1024;
        }
    }
    return g_dev;
}

struct Knob {
    const char* key;
    std::atomic<int> value;
};
static Knob g_knobs[] = {
    {"gemv_wgs_per_cu", {-1}},
    {"gemv_even_grid", {-1}},
    {"gemv_halves", {-1}},
    {"gemv_mfma_from", {-1}},
    {"gemv_five_waves", {-1}},
    {"gemv_no_mfma", {-1}},
    {"mfma_wgs_per_cu", {-1}},
    {"mfma_classic", {-1}},
    {"mfma_lds", {-1}},
    {"mfma_lds_norm", {-1}},
    {"mfma_tile_rows", {-1}},
    {"mfma_stream_x", {-1}},
    {"mfma_direct", {-1}},
    {"mfma_direct_grid", {-1}},
    {"p12_pair_table", {-1}},
    {"moe_grouped", {-1}},
    {"attn_heads_per_wg", {-1}},
    {"attn_merge_few", {-1}},
    {"attn_mfma", {-1}},
    {"attn_rows_fused", {-1}},
};

int tuning(const char* key) {
    for (Knob& k : g_knobs)
        if (std::strcmp(k.key, key) == 0) return k.value.load(std::memory_order_relaxed);
    return -1;
}

}  // namespace btb

using namespace btb;

extern "C" {

int32_t btb_hip_init(int32_t device) {
    if (device < 0) return ERR_DOMAIN;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return hip_status(e, "hipSetDevice");
    {
        std::lock_guard<std::mutex> hold(g_dev_lock);
        const int32_t rc = bind_current();
        if (rc != OK) return rc;
    }
    return attn_static_bind();
}

const char* btb_hip_arch(void) { return "gfx950"; }

int32_t btb_hip_sms(void) { return device_info().cus; }

const char* btb_hip_last_error(void) { return g_err; }

int32_t btb_hip_set_tuning(const char* key, int32_t value) {
    if (key == nullptr) return ERR_NULL;
    for (Knob& k : g_knobs)
        if (std::strcmp(k.key, key) == 0) {
            k.value.store(value < 0 ? -1 : value, std::memory_order_relaxed);
            return OK;
        }
    set_error("unknown tuning key");
    return ERR_DOMAIN;
}

}  // extern "C"
