// Test double: an IComputeBackend over plain host memory that reports
// BackendType::CPU.  It exists so the host-side bookkeeping (tensors, block
// tables, pools, the registry) can be exercised on a machine without a GPU.
// It is not part of the library and computes nothing.
#pragma once

#include <cstring>
#include <unordered_map>
#include <vector>

#include "granite/backend.h"

namespace hosttest {

class HostMemoryBackend final : public granite::IComputeBackend {
    using Error = granite::Error;
    using ErrorCode = granite::ErrorCode;
    template <typename T>
    using Result = granite::Result<T>;

  public:
    size_t max_buffer = size_t(1) << 30;

    Result<void> initialize() override {
        up_ = true;
        return {};
    }
    void shutdown() override {
        up_ = false;
        store_.clear();
    }
    bool is_initialized() const override { return up_; }
    granite::DeviceCapabilities get_capabilities() const override {
        granite::DeviceCapabilities c;
        c.name = "host-memory test double";
        c.max_buffer_size = max_buffer;
        return c;
    }
    granite::BackendType get_type() const override { return granite::BackendType::CPU; }

    Result<granite::BufferHandle> create_buffer(const granite::BufferDesc& d) override {
        if (!up_) return Error(ErrorCode::BackendNotInitialized, "down");
        granite::BufferHandle h{next_++};
        store_[h.id].assign(d.size, 0);
        return h;
    }
    void destroy_buffer(granite::BufferHandle h) override { store_.erase(h.id); }
    Result<void*> map_buffer(granite::BufferHandle h) override {
        auto it = store_.find(h.id);
        if (it == store_.end()) return Error(ErrorCode::InvalidArgument, "unknown handle");
        return static_cast<void*>(it->second.data());
    }
    void unmap_buffer(granite::BufferHandle) override {}
    Result<void> write_buffer(granite::BufferHandle h, const void* p, size_t n, size_t off) override {
        auto it = store_.find(h.id);
        if (it == store_.end() || off + n > it->second.size())
            return Error(ErrorCode::InvalidArgument, "bad write");
        std::memcpy(it->second.data() + off, p, n);
        return {};
    }
    Result<void> read_buffer(granite::BufferHandle h, void* p, size_t n, size_t off) override {
        auto it = store_.find(h.id);
        if (it == store_.end() || off + n > it->second.size())
            return Error(ErrorCode::InvalidArgument, "bad read");
        std::memcpy(p, it->second.data() + off, n);
        return {};
    }
    Result<void> copy_buffer(granite::BufferHandle s, granite::BufferHandle d, size_t n, size_t so,
                             size_t dof) override {
        auto a = store_.find(s.id), b = store_.find(d.id);
        if (a == store_.end() || b == store_.end() || so + n > a->second.size() ||
            dof + n > b->second.size())
            return Error(ErrorCode::InvalidArgument, "bad copy");
        std::memmove(b->second.data() + dof, a->second.data() + so, n);
        return {};
    }
    Result<granite::PipelineHandle> create_pipeline(const granite::PipelineDesc&) override {
        return Error(ErrorCode::NotImplemented, "test double");
    }
    void destroy_pipeline(granite::PipelineHandle) override {}
    Result<void> begin_commands() override { return {}; }
    Result<void> bind_pipeline(granite::PipelineHandle) override { return {}; }
    Result<void> bind_buffer(uint32_t, granite::BufferHandle, size_t) override { return {}; }
    Result<void> set_push_constants(const void*, size_t) override { return {}; }
    Result<void> dispatch(uint32_t, uint32_t, uint32_t) override { return {}; }
    Result<void> end_commands() override { return {}; }
    Result<void> submit() override { return {}; }
    Result<void> wait_for_completion() override { return {}; }
    Result<granite::FenceHandle> create_fence() override { return granite::FenceHandle{next_++}; }
    Result<void> wait_fence(granite::FenceHandle, uint64_t) override { return {}; }
    void destroy_fence(granite::FenceHandle) override {}

    size_t live_buffers() const { return store_.size(); }

  private:
    bool up_ = false;
    uint64_t next_ = 1;
    std::unordered_map<uint64_t, std::vector<unsigned char>> store_;
};

}  // namespace hosttest
