// HipBackend: IComputeBackend for one MI355X through the C ABI.
//
// Memory kinds
//   Device   hipMalloc'd HBM; not mappable.
//   Shared   pinned host memory; the same pointer is valid on host and device.
//   Managed  HBM plus a pinned host mirror that is created on the first
//            map_buffer().  map copies HBM -> mirror, the last unmap copies the
//            mirror back, so host code written for unified memory (map, edit,
//            unmap) keeps working; kernels always see the HBM copy.
#include "granite/hip_backend.h"

#include <cstring>
#include <mutex>
#include <unordered_map>

#include "granite/hip_compute.h"
#include "granite/operators.h"
#include "granite_hip.h"

namespace granite {
namespace {

struct Allocation {
    void* device = nullptr;   // what kernels read (pinned host pointer for Shared)
    void* mirror = nullptr;   // Managed only, lazily created
    size_t size = 0;
    MemoryType kind = MemoryType::Device;
    int map_count = 0;
};

class HipBackend final : public IComputeBackend {
  public:
    ~HipBackend() override { shutdown(); }

    Result<void> initialize() override {
        if (ready_) return {};
        auto up = compute_.initialize();
        if (!up.ok()) return up.error();
        granite_hip_device_info info{};
        GRANITE_TRY(hip_status_to_result(granite_hip_get_device_info(&info), "device info"));
        name_ = info.name[0] ? info.name : info.arch;  // some drivers leave the marketing name empty
        caps_.name = name_.c_str();
        caps_.max_buffer_size = info.max_buffer_size;
        caps_.max_threadgroup_size = static_cast<size_t>(info.max_threads_per_block);
        caps_.shared_memory_size = info.shared_memory_per_block;
        caps_.simd_width = static_cast<uint32_t>(info.wavefront_size);
        caps_.supports_fp16 = caps_.supports_bf16 = caps_.supports_int8 = true;
        caps_.supports_int4 = false;
        caps_.supports_simd_groups = true;
        ready_ = true;
        return {};
    }

    void shutdown() override {
        if (!ready_) return;
        (void)granite_hip_sync();
        for (auto& [id, a] : buffers_) release(a);
        buffers_.clear();
        for (auto& [id, ev] : fences_) (void)granite_hip_event_destroy(ev);
        fences_.clear();
        ready_ = false;  // the library context stays up: other users may share it
    }

    bool is_initialized() const override { return ready_; }
    DeviceCapabilities get_capabilities() const override { return caps_; }
    BackendType get_type() const override { return BackendType::HIP; }

    Result<BufferHandle> create_buffer(const BufferDesc& desc) override {
        if (!ready_) return Error(ErrorCode::BackendNotInitialized, "HIP backend not initialized");
        if (desc.size == 0) return Error(ErrorCode::InvalidArgument, "Buffer size must be positive");
        Allocation a;
        a.size = desc.size;
        a.kind = desc.memory_type;
        const int kind = desc.memory_type == MemoryType::Shared ? GRANITE_HIP_MEM_SHARED
                                                                : GRANITE_HIP_MEM_DEVICE;
        int status = granite_hip_malloc(&a.device, desc.size, kind);
        if (status != GRANITE_HIP_OK)
            return Error(ErrorCode::AllocationFailed,
                         std::string("HIP allocation failed: ") + granite_hip_error_string(status));
        std::lock_guard<std::mutex> lock(mutex_);
        BufferHandle h{next_id_++};
        buffers_[h.id] = a;
        return h;
    }

    void destroy_buffer(BufferHandle handle) override {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = buffers_.find(handle.id);
        if (it == buffers_.end()) return;
        (void)granite_hip_sync();  // no kernel may still be using it
        release(it->second);
        buffers_.erase(it);
    }

    Result<void*> map_buffer(BufferHandle handle) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* a = find(handle);
        if (!a) return Error(ErrorCode::InvalidArgument, "Unknown buffer handle");
        if (a->kind == MemoryType::Device)
            return Error(ErrorCode::InvalidArgument, "Device-only buffers cannot be mapped");
        if (a->kind == MemoryType::Shared) {
            GRANITE_TRY(hip_status_to_result(granite_hip_sync(), "sync before map"));
            a->map_count++;
            return a->device;
        }
        if (!a->mirror) {
            int status = granite_hip_malloc(&a->mirror, a->size, GRANITE_HIP_MEM_SHARED);
            if (status != GRANITE_HIP_OK)
                return Error(ErrorCode::AllocationFailed, "No host memory for the buffer mirror");
        }
        if (a->map_count == 0)
            GRANITE_TRY(hip_status_to_result(granite_hip_memcpy_d2h(a->mirror, a->device, a->size),
                                             "map_buffer download"));
        a->map_count++;
        return a->mirror;
    }

    void unmap_buffer(BufferHandle handle) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* a = find(handle);
        if (!a || a->map_count == 0) return;
        if (--a->map_count == 0 && a->kind == MemoryType::Managed)
            (void)granite_hip_memcpy_h2d(a->device, a->mirror, a->size);
    }

    Result<void> write_buffer(BufferHandle handle, const void* data, size_t size,
                              size_t offset) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* a = find(handle);
        if (!a) return Error(ErrorCode::InvalidArgument, "Unknown buffer handle");
        if (!data) return Error(ErrorCode::NullPointer, "Null source pointer");
        if (offset > a->size || size > a->size - offset)
            return Error(ErrorCode::BufferTooSmall, "Write exceeds buffer size");
        if (a->kind == MemoryType::Shared) {
            GRANITE_TRY(hip_status_to_result(granite_hip_sync(), "sync before write"));
            std::memcpy(static_cast<char*>(a->device) + offset, data, size);
            return {};
        }
        if (a->map_count > 0 && a->mirror)  // keep an open mapping coherent
            std::memcpy(static_cast<char*>(a->mirror) + offset, data, size);
        return hip_status_to_result(
            granite_hip_memcpy_h2d(static_cast<char*>(a->device) + offset, data, size),
            "write_buffer");
    }

    Result<void> read_buffer(BufferHandle handle, void* data, size_t size, size_t offset) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* a = find(handle);
        if (!a) return Error(ErrorCode::InvalidArgument, "Unknown buffer handle");
        if (!data) return Error(ErrorCode::NullPointer, "Null destination pointer");
        if (offset > a->size || size > a->size - offset)
            return Error(ErrorCode::BufferTooSmall, "Read exceeds buffer size");
        if (a->kind == MemoryType::Shared) {
            GRANITE_TRY(hip_status_to_result(granite_hip_sync(), "sync before read"));
            std::memcpy(data, static_cast<const char*>(a->device) + offset, size);
            return {};
        }
        return hip_status_to_result(
            granite_hip_memcpy_d2h(data, static_cast<const char*>(a->device) + offset, size),
            "read_buffer");
    }

    Result<void> copy_buffer(BufferHandle src, BufferHandle dst, size_t size, size_t src_offset,
                             size_t dst_offset) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* s = find(src);
        Allocation* d = find(dst);
        if (!s || !d) return Error(ErrorCode::InvalidArgument, "Unknown buffer handle");
        if (src_offset > s->size || size > s->size - src_offset || dst_offset > d->size ||
            size > d->size - dst_offset)
            return Error(ErrorCode::BufferTooSmall, "Copy exceeds buffer size");
        return hip_status_to_result(
            granite_hip_memcpy_d2d(static_cast<char*>(d->device) + dst_offset,
                                   static_cast<const char*>(s->device) + src_offset, size),
            "copy_buffer");
    }

    void* get_native_buffer(BufferHandle handle) override {
        std::lock_guard<std::mutex> lock(mutex_);
        Allocation* a = find(handle);
        return a ? a->device : nullptr;
    }
    void* get_native_queue() override { return granite_hip_get_stream(); }

    // Kernels are compiled ahead of time; there is no run-time shader pipeline.
    Result<PipelineHandle> create_pipeline(const PipelineDesc&) override {
        return Error(ErrorCode::NotImplemented, "HIP backend has no shader-source pipelines");
    }
    void destroy_pipeline(PipelineHandle) override {}
    Result<void> begin_commands() override { return {}; }
    Result<void> bind_pipeline(PipelineHandle) override { return not_a_pipeline_backend(); }
    Result<void> bind_buffer(uint32_t, BufferHandle, size_t) override {
        return not_a_pipeline_backend();
    }
    Result<void> set_push_constants(const void*, size_t) override {
        return not_a_pipeline_backend();
    }
    Result<void> dispatch(uint32_t, uint32_t, uint32_t) override { return not_a_pipeline_backend(); }
    Result<void> end_commands() override { return {}; }
    Result<void> submit() override { return {}; }  // launches are enqueued as they are made
    Result<void> wait_for_completion() override {
        if (!ready_) return Error(ErrorCode::BackendNotInitialized, "HIP backend not initialized");
        return hip_status_to_result(granite_hip_sync(), "wait_for_completion");
    }

    // A fence marks the work enqueued so far on the launch stream.
    Result<FenceHandle> create_fence() override {
        if (!ready_) return Error(ErrorCode::BackendNotInitialized, "HIP backend not initialized");
        void* ev = nullptr;
        GRANITE_TRY(hip_status_to_result(granite_hip_event_create(&ev), "create_fence"));
        auto rec = hip_status_to_result(granite_hip_event_record(ev), "create_fence record");
        if (!rec.ok()) {
            (void)granite_hip_event_destroy(ev);
            return rec.error();
        }
        std::lock_guard<std::mutex> lock(mutex_);
        FenceHandle h{next_id_++};
        fences_[h.id] = ev;
        return h;
    }
    Result<void> wait_fence(FenceHandle fence, uint64_t /*timeout_ns*/) override {
        void* ev = nullptr;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            auto it = fences_.find(fence.id);
            if (it == fences_.end()) return Error(ErrorCode::InvalidArgument, "Unknown fence");
            ev = it->second;
        }
        return hip_status_to_result(granite_hip_event_synchronize(ev), "wait_fence");
    }
    void destroy_fence(FenceHandle fence) override {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = fences_.find(fence.id);
        if (it == fences_.end()) return;
        (void)granite_hip_event_destroy(it->second);
        fences_.erase(it);
    }

  private:
    static Result<void> not_a_pipeline_backend() {
        return Error(ErrorCode::NotImplemented, "HIP backend has no shader-source pipelines");
    }
    Allocation* find(BufferHandle h) {
        auto it = buffers_.find(h.id);
        return it == buffers_.end() ? nullptr : &it->second;
    }
    static void release(Allocation& a) {
        (void)granite_hip_free(a.device, a.kind == MemoryType::Shared ? GRANITE_HIP_MEM_SHARED
                                                                       : GRANITE_HIP_MEM_DEVICE);
        if (a.mirror) (void)granite_hip_free(a.mirror, GRANITE_HIP_MEM_SHARED);
        a.device = a.mirror = nullptr;
    }

    HipCompute compute_;
    bool ready_ = false;
    std::string name_;
    DeviceCapabilities caps_{};
    std::mutex mutex_;
    uint64_t next_id_ = 1;
    std::unordered_map<uint64_t, Allocation> buffers_;
    std::unordered_map<uint64_t, void*> fences_;
};

}  // namespace

std::unique_ptr<IComputeBackend> create_hip_backend() { return std::make_unique<HipBackend>(); }

void* hip_device_pointer(IComputeBackend* backend, BufferHandle handle) {
    if (!backend || backend->get_type() != BackendType::HIP) return nullptr;
    return backend->get_native_buffer(handle);
}

// The factory of this library knows one backend (src/core/backend_factory.cpp:12-40
// is where the reference lists its own).
std::unique_ptr<IComputeBackend> create_backend(BackendType type) {
    initialize_operators();  // as the reference does on first backend creation (:36-37)
    return type == BackendType::HIP ? create_hip_backend() : nullptr;
}
std::unique_ptr<IComputeBackend> create_default_backend() { return create_hip_backend(); }
bool is_backend_available(BackendType type) {
    if (type != BackendType::HIP) return false;
    return get_hip_compute() != nullptr;
}

}  // namespace granite
