// Value types of the Granite API surface that the HIP backend plugs into:
// element types, backend ids, opaque handles, buffer descriptions, device
// capabilities.  Enumerator order follows the reference (include/granite/types.h:13-187)
// so that values agree; BackendType gains HIP after Talos, the way Talos itself
// was added (include/granite/types.h:93-98).
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>

namespace granite {

enum class DataType : uint8_t { FP32, FP16, BF16, INT32, INT64, INT16, INT8, UINT8, BOOL, INT4, UINT4 };

constexpr size_t dtype_size(DataType t) {
    switch (t) {
        case DataType::FP32: case DataType::INT32: return 4;
        case DataType::INT64: return 8;
        case DataType::FP16: case DataType::BF16: case DataType::INT16: return 2;
        default: return 1;  // INT8, UINT8, BOOL and the packed 4-bit types (two per byte)
    }
}
constexpr bool dtype_is_float(DataType t) {
    return t == DataType::FP32 || t == DataType::FP16 || t == DataType::BF16;
}
constexpr bool dtype_is_quantized(DataType t) {
    return t == DataType::INT4 || t == DataType::UINT4 || t == DataType::INT8;
}
constexpr const char* dtype_name(DataType t) {
    constexpr const char* names[] = {"fp32", "fp16", "bf16", "int32", "int64", "int16",
                                     "int8", "uint8", "bool", "int4", "uint4"};
    return static_cast<size_t>(t) < sizeof(names) / sizeof(names[0]) ? names[static_cast<size_t>(t)]
                                                                     : "unknown";
}

enum class MemoryLayout : uint8_t { RowMajor, ColMajor, NCHW, NHWC, Custom };

enum class BackendType : uint8_t { CPU, Metal, Vulkan, Talos, HIP };

constexpr const char* backend_name(BackendType t) {
    switch (t) {
        case BackendType::CPU: return "CPU";
        case BackendType::Metal: return "Metal";
        case BackendType::Vulkan: return "Vulkan";
        case BackendType::Talos: return "Talos";
        case BackendType::HIP: return "HIP";
    }
    return "unknown";
}

// Opaque ids handed out by a backend; 0 is never valid.
template <int Tag>
struct Handle {
    uint64_t id = 0;
    bool valid() const { return id != 0; }
    bool operator==(const Handle& o) const { return id == o.id; }
    bool operator!=(const Handle& o) const { return id != o.id; }
};
using BufferHandle = Handle<0>;
using PipelineHandle = Handle<1>;
using FenceHandle = Handle<2>;

enum class MemoryType : uint8_t {
    Device,   // GPU only
    Shared,   // host memory the GPU can reach (uploads / downloads)
    Managed,  // CPU-mappable device data (what Tensor::allocate asks for)
};

struct BufferDesc {
    size_t size = 0;
    MemoryType memory_type = MemoryType::Device;
    bool allow_aliasing = false;
    static BufferDesc device(size_t n) { return {n, MemoryType::Device, false}; }
    static BufferDesc shared(size_t n) { return {n, MemoryType::Shared, false}; }
    static BufferDesc managed(size_t n) { return {n, MemoryType::Managed, false}; }
};

struct DeviceCapabilities {
    const char* name = nullptr;
    size_t max_buffer_size = 0;
    size_t max_threadgroup_size = 0;
    size_t shared_memory_size = 0;
    uint32_t simd_width = 0;
    bool supports_fp16 = false;
    bool supports_bf16 = false;
    bool supports_int8 = false;
    bool supports_int4 = false;
    bool supports_simd_groups = false;
};

}  // namespace granite

namespace std {
template <int Tag>
struct hash<granite::Handle<Tag>> {
    size_t operator()(const granite::Handle<Tag>& h) const { return std::hash<uint64_t>{}(h.id); }
};
}  // namespace std
