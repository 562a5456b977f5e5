// IComputeBackend: the device abstraction Granite's tensors, KV caches and
// operators are written against (reference: include/granite/backend.h:30-198).
// The HIP backend implements it in hip_backend.h; create_backend(BackendType::HIP)
// returns it, the way create_talos_backend_granite() is wired in
// src/core/backend_factory.cpp:29-31, 62-68.
#pragma once

#include <memory>
#include <string>

#include "granite/error.h"
#include "granite/types.h"

namespace granite {

struct PipelineDesc {
    std::string shader_source;
    std::string entry_point = "main";
    uint32_t threadgroup_size_x = 0, threadgroup_size_y = 0, threadgroup_size_z = 0;
};

class IComputeBackend {
  public:
    virtual ~IComputeBackend() = default;

    // lifecycle
    virtual Result<void> initialize() = 0;
    virtual void shutdown() = 0;
    [[nodiscard]] virtual bool is_initialized() const = 0;

    // device info
    [[nodiscard]] virtual DeviceCapabilities get_capabilities() const = 0;
    [[nodiscard]] virtual BackendType get_type() const = 0;

    // buffers
    virtual Result<BufferHandle> create_buffer(const BufferDesc& desc) = 0;
    virtual Result<BufferHandle> create_buffer_from_host(const void* data, const BufferDesc& desc) {
        if (!data) return Error(ErrorCode::InvalidArgument, "Null host buffer");
        auto made = create_buffer(desc);
        if (!made.ok()) return made.error();
        auto written = write_buffer(made.value(), data, desc.size);
        if (!written.ok()) {
            destroy_buffer(made.value());
            return written.error();
        }
        return made;
    }
    virtual void destroy_buffer(BufferHandle handle) = 0;
    virtual Result<void*> map_buffer(BufferHandle handle) = 0;
    virtual void unmap_buffer(BufferHandle handle) = 0;
    virtual Result<void> write_buffer(BufferHandle handle, const void* data, size_t size,
                                      size_t offset = 0) = 0;
    virtual Result<void> read_buffer(BufferHandle handle, void* data, size_t size,
                                     size_t offset = 0) = 0;
    virtual Result<void> copy_buffer(BufferHandle src, BufferHandle dst, size_t size,
                                     size_t src_offset = 0, size_t dst_offset = 0) = 0;
    virtual void* get_native_buffer(BufferHandle) { return nullptr; }
    virtual void* get_native_device() { return nullptr; }
    virtual void* get_native_physical_device() { return nullptr; }
    virtual void* get_native_queue() { return nullptr; }
    virtual uint32_t get_native_queue_family() { return 0; }

    // generic pipelines / command recording (shader-source backends only)
    virtual Result<PipelineHandle> create_pipeline(const PipelineDesc& desc) = 0;
    virtual void destroy_pipeline(PipelineHandle handle) = 0;
    virtual Result<void> begin_commands() = 0;
    virtual Result<void> bind_pipeline(PipelineHandle pipeline) = 0;
    virtual Result<void> bind_buffer(uint32_t index, BufferHandle buffer, size_t offset = 0) = 0;
    virtual Result<void> set_push_constants(const void* data, size_t size) = 0;
    virtual Result<void> dispatch(uint32_t groups_x, uint32_t groups_y = 1,
                                  uint32_t groups_z = 1) = 0;
    virtual Result<void> end_commands() = 0;
    virtual Result<void> submit() = 0;
    virtual Result<void> wait_for_completion() = 0;

    // fences
    virtual Result<FenceHandle> create_fence() = 0;
    virtual Result<void> wait_fence(FenceHandle fence, uint64_t timeout_ns = UINT64_MAX) = 0;
    virtual void destroy_fence(FenceHandle fence) = 0;
};

std::unique_ptr<IComputeBackend> create_backend(BackendType type);
std::unique_ptr<IComputeBackend> create_default_backend();
bool is_backend_available(BackendType type);

}  // namespace granite
