// HipBackend: IComputeBackend over libgranite_hip.so for one MI355X.
// Plays the part MetalBackend / TalosBackendGranite play in the reference
// (src/core/backend_factory.cpp:17-31): buffers, copies, fences.  The generic
// shader-pipeline calls answer NotImplemented: kernels are compiled ahead of
// time and reached through HipCompute and the registered operators.
#pragma once

#include <memory>

#include "granite/backend.h"

namespace granite {

// nullptr is never returned; initialize() reports whether a gfx950 GPU is usable.
std::unique_ptr<IComputeBackend> create_hip_backend();

// Device pointer behind a buffer of a HIP backend (nullptr for other backends
// or unknown handles).  Shorthand for get_native_buffer().
void* hip_device_pointer(IComputeBackend* backend, BufferHandle handle);

}  // namespace granite
