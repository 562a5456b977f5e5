// (op, backend) -> factory table.
#include <algorithm>

#include "granite/operators.h"

namespace granite {

const char* op_type_name(OpType op) {
    static constexpr const char* names[] = {
        "Reshape", "Transpose", "Concat", "Split", "Slice", "Gather",
        "Add", "Sub", "Mul", "Div", "Neg", "Sqrt", "Exp", "Log", "Pow",
        "ReLU", "GELU", "SiLU", "Sigmoid", "Tanh", "Softmax",
        "MatMul", "BatchMatMul", "QuantizedMatMul",
        "Conv2D", "DepthwiseConv2D", "ConvTranspose2D",
        "LayerNorm", "RMSNorm", "BatchNorm", "GroupNorm",
        "MaxPool2D", "AvgPool2D", "GlobalAvgPool", "AdaptiveAvgPool",
        "ScaledDotProductAttention", "MultiHeadAttention",
        "Embedding", "RoPE", "CausalMask", "Quantize", "Dequantize", "Custom"};
    const auto i = static_cast<size_t>(op);
    return i < sizeof(names) / sizeof(names[0]) ? names[i] : "Unknown";
}

OperatorRegistry& OperatorRegistry::instance() {
    static OperatorRegistry registry;
    return registry;
}

void OperatorRegistry::register_op(OpType op, BackendType backend, OperatorFactory factory) {
    factories_[key(op, backend)] = std::move(factory);
}

std::unique_ptr<IOperator> OperatorRegistry::create(OpType op, BackendType backend) const {
    auto it = factories_.find(key(op, backend));
    if (it == factories_.end() && backend != BackendType::CPU)
        it = factories_.find(key(op, BackendType::CPU));
    return it == factories_.end() ? nullptr : it->second();
}

bool OperatorRegistry::has_implementation(OpType op, BackendType backend) const {
    return factories_.count(key(op, backend)) != 0;
}

std::vector<OpType> OperatorRegistry::get_ops_for_backend(BackendType backend) const {
    std::vector<OpType> ops;
    for (const auto& entry : factories_)
        if ((entry.first & 0xff) == static_cast<uint64_t>(backend))
            ops.push_back(static_cast<OpType>(entry.first >> 8));
    std::sort(ops.begin(), ops.end());
    return ops;
}

void initialize_operators() { register_hip_operators(); }

}  // namespace granite
