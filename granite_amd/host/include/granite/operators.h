// Operator plug-in surface (reference: include/granite/operators.h:20-290,
// src/core/operator_registry.cpp:10-54): OpType, Attributes, OpContext,
// IOperator and the (op, backend) -> factory registry.  The HIP backend
// registers ScaledDotProductAttention through register_hip_operators(), the
// same hook shape as register_metal_operators().
#pragma once

#include <functional>
#include <memory>
#include <string>
#include <unordered_map>
#include <variant>
#include <vector>

#include "granite/tensor.h"

namespace granite {

// Same order as the reference, so enumerator values agree.
enum class OpType : uint32_t {
    Reshape, Transpose, Concat, Split, Slice, Gather,
    Add, Sub, Mul, Div, Neg, Sqrt, Exp, Log, Pow,
    ReLU, GELU, SiLU, Sigmoid, Tanh, Softmax,
    MatMul, BatchMatMul, QuantizedMatMul,
    Conv2D, DepthwiseConv2D, ConvTranspose2D,
    LayerNorm, RMSNorm, BatchNorm, GroupNorm,
    MaxPool2D, AvgPool2D, GlobalAvgPool, AdaptiveAvgPool,
    ScaledDotProductAttention, MultiHeadAttention,
    Embedding, RoPE, CausalMask,
    Quantize, Dequantize,
    Custom,
};

const char* op_type_name(OpType op);

using AttrValue = std::variant<int64_t, double, bool, std::string, std::vector<int64_t>,
                               std::vector<double>>;

class Attributes {
  public:
    void set(const std::string& key, AttrValue value) { values_[key] = std::move(value); }
    bool has(const std::string& key) const { return values_.count(key) != 0; }
    // A missing key or a value of another alternative yields the fallback.
    template <typename T>
    T get(const std::string& key, T fallback = T{}) const {
        auto it = values_.find(key);
        if (it == values_.end()) return fallback;
        const T* held = std::get_if<T>(&it->second);
        return held ? *held : fallback;
    }

  private:
    std::unordered_map<std::string, AttrValue> values_;
};

struct OpContext {
    IComputeBackend* backend = nullptr;
    std::vector<Tensor> inputs;
    std::vector<Tensor> outputs;
    Attributes attrs;

    const Tensor& input(size_t i) const { return inputs.at(i); }
    Tensor& output(size_t i) { return outputs.at(i); }
    size_t num_inputs() const { return inputs.size(); }
    size_t num_outputs() const { return outputs.size(); }
};

class IOperator {
  public:
    virtual ~IOperator() = default;
    [[nodiscard]] virtual OpType type() const = 0;
    [[nodiscard]] virtual Result<void> validate(const OpContext& ctx) const = 0;
    [[nodiscard]] virtual Result<std::vector<std::vector<int64_t>>> infer_shapes(
        const OpContext& ctx) const = 0;
    [[nodiscard]] virtual Result<void> execute(OpContext& ctx) = 0;
    [[nodiscard]] virtual bool can_fuse_with(OpType) const { return false; }
};

using OperatorFactory = std::function<std::unique_ptr<IOperator>()>;

class OperatorRegistry {
  public:
    static OperatorRegistry& instance();
    // A later registration for the same (op, backend) replaces the earlier one.
    void register_op(OpType op, BackendType backend, OperatorFactory factory);
    // Falls back to the CPU factory of `op`; nullptr when neither exists.
    [[nodiscard]] std::unique_ptr<IOperator> create(OpType op, BackendType backend) const;
    [[nodiscard]] bool has_implementation(OpType op, BackendType backend) const;
    [[nodiscard]] std::vector<OpType> get_ops_for_backend(BackendType backend) const;

  private:
    OperatorRegistry() = default;
    static uint64_t key(OpType op, BackendType backend) {
        return (static_cast<uint64_t>(op) << 8) | static_cast<uint64_t>(backend);
    }
    std::unordered_map<uint64_t, OperatorFactory> factories_;
};

#define GRANITE_REGISTER_OP(op_type, backend_type, cls)                                  \
    static bool _granite_reg_##op_type##_##backend_type = [] {                           \
        ::granite::OperatorRegistry::instance().register_op(                             \
            ::granite::OpType::op_type, ::granite::BackendType::backend_type,            \
            []() -> std::unique_ptr<::granite::IOperator> { return std::make_unique<cls>(); }); \
        return true;                                                                     \
    }()

// Registers the HIP operators (ScaledDotProductAttention); idempotent.
void register_hip_operators();
// Registers every backend compiled into this library (here: HIP).
void initialize_operators();

}  // namespace granite
