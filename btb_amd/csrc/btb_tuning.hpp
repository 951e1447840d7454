// Launch tuning shared by the kernels' host entry points: the device's compute-unit count and a small table of
// integer knobs a caller may override (`btb_hip_set_tuning`), each with a default picked by measurement on MI355X.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace btb {

struct DeviceInfo {
    int cus = 0;          // compute units of the current device
    int lds_bytes = 0;    // LDS a workgroup may take
    bool ready = false;
};

// the current device's facts, read once per process (one GPU per process)
const DeviceInfo& device_info();

// a knob's value: -1 where the caller has not set one
int tuning(const char* key);

// maps a HIP status to the C ABI's code, remembering the message for btb_hip_last_error
int32_t hip_status(hipError_t e, const char* what);
void set_error(const char* msg);

}  // namespace btb
