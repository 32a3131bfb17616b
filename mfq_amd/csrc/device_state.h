// One-time set-up per device, shared by every entry point: the SwiGLU sigmoid table and the dynamic-LDS
// limits of the kernels that need more than the default 64 KB.
#pragma once

#include <stdint.h>

namespace mfq_amd {

struct DeviceState {
    const uint16_t* sigmoid_table;   // [65536] half(sigmoid(g)) indexed by the bits of the half g, sigmoid in double
    void* static_scratch;            // this device's copy of the library's static scratch array
};

// State of the current device.  The first call on a device allocates, copies and synchronises (and must
// therefore not happen inside a stream capture); later calls only read.  Safe to call from several threads.
const DeviceState& device_state();
// The same, or null when the device has not been set up yet (never allocates).
const DeviceState* device_state_if_ready();

// Raise the dynamic-LDS limits of the kernels of one translation unit on the current device.
void raise_routing_limits();
void raise_prefill_limits();

// IEEE binary64 -> binary16 with one rounding; binary16 -> binary32.
uint16_t double_to_half(double value);
float half_to_float_host(uint16_t h);

}  // namespace mfq_amd
