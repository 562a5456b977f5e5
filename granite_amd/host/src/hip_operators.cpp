// HipAttentionOp: OpType::ScaledDotProductAttention on BackendType::HIP.
//
// Stands where MetalAttentionOp stands in the reference
// (src/operators/metal/metal_operators.mm:1226-1320): inputs Q, K, V, one output
// shaped like Q, attributes `scale` (default 1/sqrt(D)) and `start_pos`
// (default 0), key k visible to query q iff k <= q + start_pos
// (metal_operators.mm:640-641).  Unlike that operator it works on the device
// buffers in place (no map/copy round trip) and accepts head dimensions.  The
// kernels exist for head sizes 64 and 128; any other size up to 128 is presented
// to them zero-padded (zero columns add nothing to a score and give zero output
// columns, which are sliced off again), so the reference's small test tensors
// (head size 4, tests/test_vulkan.cpp:353-482) go through unchanged.  Shapes:
//   Q, out  [seq_q, D] | [H, seq_q, D] | [B, H, seq_q, D]   FP16 or FP32
//   K, V    [seq_kv, D] | [Hkv, seq_kv, D] | [B, Hkv, seq_kv, D]   FP16 or FP32
// with H a multiple of Hkv (grouped-query attention).  The kernels read K and V as halves (the
// KV cache type); float K and V -- what the reference's operator tests allocate
// (tests/test_vulkan.cpp:372-374) -- are first rounded to nearest into half temporaries, as the
// reference's GPU kernels round what they store (metal_shaders_attention.h:124).  The extra attribute
// `causal` (bool, default true) switches the mask off, which is what the
// Vulkan operator computes (src/operators/vulkan/vulkan_operators.cpp:392-397).
#include <cmath>
#include <mutex>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite/operators.h"
#include "granite_hip.h"

namespace granite {
namespace {

struct AttnDims {
    int64_t batch = 1, heads = 1, seq = 0, dim = 0;
};

Result<AttnDims> split_dims(const Tensor& t, const char* what) {
    AttnDims d;
    const size_t n = t.ndim();
    if (n < 2 || n > 4)
        return Error(ErrorCode::InvalidShape, std::string(what) + " must have 2 to 4 dimensions");
    d.dim = t.size(-1);
    d.seq = t.size(-2);
    if (n >= 3) d.heads = t.size(-3);
    if (n == 4) d.batch = t.size(0);
    return d;
}

class HipAttentionOp final : public IOperator {
  public:
    OpType type() const override { return OpType::ScaledDotProductAttention; }

    Result<void> validate(const OpContext& ctx) const override {
        if (ctx.num_inputs() < 3)
            return Error(ErrorCode::InvalidArgument, "Attention requires 3 inputs (Q, K, V)");
        const Tensor& Q = ctx.inputs[0];
        const Tensor& K = ctx.inputs[1];
        const Tensor& V = ctx.inputs[2];
        GRANITE_TRY_ASSIGN(q, split_dims(Q, "Q"));
        GRANITE_TRY_ASSIGN(k, split_dims(K, "K"));
        GRANITE_TRY_ASSIGN(v, split_dims(V, "V"));
        if (Q.ndim() != K.ndim() || K.ndim() != V.ndim())
            return Error(ErrorCode::ShapeMismatch, "Q, K and V must have the same rank");
        if (k.dim != q.dim || v.dim != q.dim || v.seq != k.seq || v.heads != k.heads ||
            k.batch != q.batch || v.batch != q.batch)
            return Error(ErrorCode::ShapeMismatch, "Q, K and V shapes do not agree");
        if (k.heads <= 0 || q.heads % k.heads != 0)
            return Error(ErrorCode::ShapeMismatch, "Query heads must be a multiple of KV heads");
        if (Q.dtype() != DataType::FP16 && Q.dtype() != DataType::FP32)
            return Error(ErrorCode::DTypeMismatch, "Q must be FP16 or FP32");
        if ((K.dtype() != DataType::FP16 && K.dtype() != DataType::FP32) || V.dtype() != K.dtype())
            return Error(ErrorCode::DTypeMismatch, "K and V must both be FP16 (the KV cache type) or both FP32");
        if (!Q.is_contiguous() || !K.is_contiguous() || !V.is_contiguous())
            return Error(ErrorCode::InvalidArgument, "Q, K and V must be contiguous");
        if (q.dim < 1 || q.dim > 128)
            return Error(ErrorCode::NotImplemented, "HipAttentionOp serves head_dim 1 .. 128");
        return {};
    }

    Result<std::vector<std::vector<int64_t>>> infer_shapes(const OpContext& ctx) const override {
        if (ctx.num_inputs() < 1) return Error(ErrorCode::InvalidArgument, "Attention needs Q");
        auto s = ctx.inputs[0].shape();
        return std::vector<std::vector<int64_t>>{std::vector<int64_t>(s.begin(), s.end())};
    }

    Result<void> execute(OpContext& ctx) override {
        GRANITE_TRY(validate(ctx));
        if (!ctx.backend || ctx.backend->get_type() != BackendType::HIP)
            return Error(ErrorCode::BackendNotSupported, "HipAttentionOp needs a HIP backend");
        if (ctx.num_outputs() < 1) return Error(ErrorCode::InvalidArgument, "Attention needs an output");
        const Tensor& Q = ctx.inputs[0];
        const Tensor& K = ctx.inputs[1];
        const Tensor& V = ctx.inputs[2];
        Tensor& out = ctx.outputs[0];
        if (out.dtype() != Q.dtype() || out.numel() != Q.numel() || !out.is_contiguous())
            return Error(ErrorCode::ShapeMismatch, "Output must match Q in shape and dtype");

        const AttnDims q = split_dims(Q, "Q").value();
        const AttnDims k = split_dims(K, "K").value();
        const double scale =
            ctx.attrs.get<double>("scale", 1.0 / std::sqrt(static_cast<double>(q.dim)));
        const int64_t start_pos = ctx.attrs.get<int64_t>("start_pos", 0);
        const bool causal = ctx.attrs.get<bool>("causal", true);
        if (start_pos < 0) return Error(ErrorCode::InvalidArgument, "start_pos must be >= 0");

        auto base = [&](const Tensor& t) -> char* {
            auto* p = static_cast<char*>(hip_device_pointer(ctx.backend, t.buffer()));
            return p ? p + t.buffer_offset() : nullptr;
        };
        char* q_ptr = base(Q);
        char* k_ptr = base(K);
        char* v_ptr = base(V);
        char* o_ptr = base(out);
        if (!q_ptr || !k_ptr || !v_ptr || !o_ptr)
            return Error(ErrorCode::InvalidArgument, "Tensor buffers do not belong to the HIP backend");

        const int dtype = Q.dtype() == DataType::FP16 ? GRANITE_HIP_F16 : GRANITE_HIP_F32;
        const size_t q_esz = dtype_size(Q.dtype());
        // head sizes without a kernel: zero-padded copies of Q, K and V, and a padded output
        const int64_t dim = q.dim == 64 || q.dim == 128 ? q.dim : (q.dim < 64 ? 64 : 128);
        const bool padded = dim != q.dim;
        const uint64_t q_rows = uint64_t(q.batch * q.heads * q.seq), kv_rows = uint64_t(k.batch * k.heads * k.seq);
        BufferHandle tmp[6] = {};  // Q, K, V, out (padded); K, V as halves
        auto release = [&] {
            for (BufferHandle& h : tmp)
                if (h.valid()) ctx.backend->destroy_buffer(h);
        };
        if (K.dtype() == DataType::FP32) {
            // [B, Hkv, seq_kv, D] float -> the same layout in halves: per batch entry an append
            // into a "cache" of exactly seq_kv rows per head, starting at row 0
            Result<void> status;
            for (int i = 4; i < 6 && status.ok(); ++i) {
                auto made = ctx.backend->create_buffer(BufferDesc::device(kv_rows * q.dim * sizeof(uint16_t)));
                if (!made.ok()) status = made.error();
                else tmp[i] = made.value();
            }
            char* kh = status.ok() ? static_cast<char*>(hip_device_pointer(ctx.backend, tmp[4])) : nullptr;
            char* vh = status.ok() ? static_cast<char*>(hip_device_pointer(ctx.backend, tmp[5])) : nullptr;
            const size_t batch_elems = size_t(k.heads * k.seq * q.dim);
            for (int64_t b = 0; b < k.batch && status.ok(); ++b)
                status = hip_status_to_result(
                    granite_hip_kv_cache_append_ex(kh + b * batch_elems * sizeof(uint16_t),
                                                   vh + b * batch_elems * sizeof(uint16_t),
                                                   k_ptr + b * batch_elems * sizeof(float),
                                                   v_ptr + b * batch_elems * sizeof(float), GRANITE_HIP_F32, q.dim,
                                                   k.seq * q.dim, uint32_t(k.heads), uint32_t(q.dim), 0,
                                                   uint32_t(k.seq), uint32_t(k.seq), GRANITE_HIP_ROUND_NEAREST),
                    "granite_hip_kv_cache_append_ex");
            if (!status.ok()) {
                release();
                return status;
            }
            k_ptr = kh;
            v_ptr = vh;
        }
        const bool temporaries = padded || K.dtype() == DataType::FP32;
        if (padded) {
            const size_t bytes[4] = {q_rows * dim * q_esz, kv_rows * dim * 2, kv_rows * dim * 2, q_rows * dim * q_esz};
            char* const src[3] = {q_ptr, k_ptr, v_ptr};
            const size_t esz[3] = {q_esz, 2, 2};
            const uint64_t rows[3] = {q_rows, kv_rows, kv_rows};
            Result<void> status;
            for (int i = 0; i < 4 && status.ok(); ++i) {
                auto made = ctx.backend->create_buffer(BufferDesc::device(bytes[i]));
                if (!made.ok()) status = made.error();
                else tmp[i] = made.value();
            }
            for (int i = 0; i < 3 && status.ok(); ++i)
                status = hip_status_to_result(
                    granite_hip_copy_rows(hip_device_pointer(ctx.backend, tmp[i]), int64_t(dim * esz[i]), src[i],
                                          int64_t(q.dim * esz[i]), rows[i], uint32_t(q.dim * esz[i]),
                                          uint32_t(dim * esz[i])),
                    "granite_hip_copy_rows");
            if (!status.ok()) {
                release();
                return status;
            }
            q_ptr = static_cast<char*>(hip_device_pointer(ctx.backend, tmp[0]));
            k_ptr = static_cast<char*>(hip_device_pointer(ctx.backend, tmp[1]));
            v_ptr = static_cast<char*>(hip_device_pointer(ctx.backend, tmp[2]));
        }
        char* const result_ptr = padded ? static_cast<char*>(hip_device_pointer(ctx.backend, tmp[3])) : o_ptr;
        const size_t q_batch_bytes = size_t(q.heads * q.seq * dim) * q_esz;
        const size_t kv_batch_bytes = size_t(k.heads * k.seq * dim) * sizeof(uint16_t);

        HipCompute compute;  // stateless façade over the already initialised library
        for (int64_t b = 0; b < q.batch; ++b) {
            granite_hip_attention_args a{};
            a.q = q_ptr + b * q_batch_bytes;
            a.q_dtype = dtype;
            a.q_tok_stride = dim;
            a.q_head_stride = q.seq * dim;
            a.out = result_ptr + b * q_batch_bytes;
            a.out_dtype = dtype;
            a.out_tok_stride = dim;
            a.out_head_stride = q.seq * dim;
            a.k_cache = k_ptr + b * kv_batch_bytes;
            a.v_cache = v_ptr + b * kv_batch_bytes;
            a.max_seq = static_cast<uint32_t>(k.seq);
            a.cache_len = static_cast<uint32_t>(k.seq);
            a.mask_mode = causal ? GRANITE_HIP_MASK_CAUSAL : GRANITE_HIP_MASK_NONE;
            a.start_pos = static_cast<uint32_t>(start_pos);
            a.seq_q = static_cast<uint32_t>(q.seq);
            a.num_heads = static_cast<uint32_t>(q.heads);
            a.num_kv_heads = static_cast<uint32_t>(k.heads);
            a.head_dim = static_cast<uint32_t>(dim);
            a.scale = static_cast<float>(scale);
            if (auto launched = compute.attention(a); !launched.ok()) {
                release();
                return launched;
            }
        }
        if (temporaries) {
            Result<void> sliced;
            if (padded)
                sliced = hip_status_to_result(
                    granite_hip_copy_rows(o_ptr, int64_t(q.dim * q_esz), result_ptr, int64_t(dim * q_esz), q_rows,
                                          uint32_t(q.dim * q_esz), uint32_t(q.dim * q_esz)),
                    "granite_hip_copy_rows");
            (void)ctx.backend->wait_for_completion();  // the temporaries are released below
            release();
            return sliced;
        }
        return {};
    }
};

}  // namespace

void register_hip_operators() {
    static std::once_flag once;
    std::call_once(once, [] {
        OperatorRegistry::instance().register_op(
            OpType::ScaledDotProductAttention, BackendType::HIP,
            []() -> std::unique_ptr<IOperator> { return std::make_unique<HipAttentionOp>(); });
    });
}

}  // namespace granite
