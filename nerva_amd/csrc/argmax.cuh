// Launch interface of the device argmax / sampler workspace (argmax.hip).
#pragma once

#include "gemv_stream.cuh"

namespace nv {

uint64_t sample_workspace_bytes();
// Carves counter/part_* out of a zero-initialised workspace of sample_workspace_bytes().
void sample_bind_workspace(SampleParams &s, void *workspace);
hipError_t launch_argmax(const float *logits, uint32_t count, const SampleParams &s,
                         hipStream_t stream);

// Resolves the device address of nerva_hip_argmax_static's candidate array on the current device
// (set-up; nerva_hip_device_smoke calls it so that later calls only launch).
hipError_t argmax_static_setup();

}  // namespace nv
