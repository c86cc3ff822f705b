// Host-side state shared by the translation units that implement the handle-based entry points:
// the library's default stream, the blocking switch and the host/device classification of a pointer.
#pragma once
#include <hip/hip_runtime.h>

namespace kutacc_api {
hipStream_t default_stream();
hipStream_t stream_or_default(void *stream); // an explicit stream argument, else the default stream
bool on_device(const void *ptr);             // device or managed memory (plain and pinned host memory: false)
int finish(int rc, hipStream_t stream);      // synchronise if the library is in blocking mode; passes rc through
// Where the attention blocks may let the head kernel normalise its input rows: 0 = where it measured at least as fast
// (256 channels), 1 = wherever the kernel can, 2 = never (the "layernorm" hook of kutacc_hip_set_tuning)
int block_layernorm_mode();
} // namespace kutacc_api
