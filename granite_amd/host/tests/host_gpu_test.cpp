// GPU tests of the C++ host layer: HipBackend buffers, HipCompute, the
// registered attention operator and the KV classes, checked against the CPU
// oracle (linked as a shared library; it is the checker, never the path under
// test).  Needs an MI355X; exits with status 77 when no usable GPU is present.
#include <cmath>
#include <cstring>
#include <random>

#include "check.h"
#include "granite/chunked_prefill.h"
#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite/kv_cache.h"
#include "granite/operators.h"
#include "granite/paged_batch.h"
#include "granite/tree_verify.h"
#include "granite/rope.h"
#include "granite_hip.h"

extern "C" {
// CPU oracle (oracle/granite_oracle.c)
uint16_t go_fp32_to_fp16(float f);
float go_fp16_to_fp32(uint16_t h);
int go_kv_cache_append_f16(uint16_t* cache, const uint16_t* src, int num_kv_heads, int head_dim,
                           int current_len, int new_len, int max_seq);
void go_paged_kv_cache_append_f32(uint16_t* pool, const float* src, const int32_t* table,
                                  int num_kv_heads, int head_dim, int start_pos, int new_len,
                                  int block_size);
int go_kv_cache_append_f32(uint16_t* cache, const float* src, int num_kv_heads, int head_dim,
                           int current_len, int new_len, int max_seq);
void go_attention_paged(const float* q, const uint16_t* pool_k, const uint16_t* pool_v,
                        const int32_t* table, int block_size, float* context, float* lse, int batch,
                        int seq_len, int num_heads, int num_kv_heads, int head_dim, int total_seq,
                        int start_pos, float scale);
void go_matvec_q4k(const float* x, const uint8_t* W, float* y, int K, int N, int batch);
void go_attention_cached(const float* q, const uint16_t* cache_k, const uint16_t* cache_v,
                         float* context, float* lse, int batch, int seq_len, int num_heads,
                         int num_kv_heads, int head_dim, int total_seq, int max_seq,
                         int start_pos, float scale);
void go_batched_paged_decode(const float* q, const uint16_t* pool_k, const uint16_t* pool_v,
                             const int32_t* tables, const int32_t* seq_lens, float* out, float* lse,
                             int batch, int num_heads, int num_kv_heads, int head_dim,
                             int block_size, int max_blocks, float scale);
void go_rope_table(float* cos_out, float* sin_out, int max_seq_len, int head_dim, float theta);
int go_rope_apply(float* x, int seq_len, int num_heads, int head_dim, int start_pos, const float* cos_t,
                  const float* sin_t, int max_seq_len);
int go_attention_tree(const float* q, const uint16_t* cache_k, const uint16_t* cache_v,
                      const int32_t* table, int block_size, int max_seq, const float* k_tree,
                      const float* v_tree, const int32_t* parent, float* context, float* lse,
                      int batch, int num_nodes, int num_heads, int num_kv_heads, int head_dim,
                      int cached_len, float scale);
}

using namespace granite;

namespace {

constexpr int D = 128;
// Output tolerance of the attention path: max-abs 2e-3, max-rel 1e-2 (either one passes).
bool close_enough(const std::vector<float>& got, const std::vector<float>& want, const char* what) {
    double worst = 0;
    size_t bad = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        const double err = std::fabs(double(got[i]) - double(want[i]));
        worst = std::max(worst, err);
        if (!(err <= 2e-3 || err <= 1e-2 * std::fabs(double(want[i])))) ++bad;
    }
    std::printf("  %s: max abs err %.3g over %zu values\n", what, worst, want.size());
    return bad == 0 && got.size() == want.size();
}

std::vector<float> randn(size_t n, uint32_t seed, float scale = 1.0f) {
    std::mt19937 gen(seed);
    std::normal_distribution<float> dist(0.0f, scale);
    std::vector<float> v(n);
    for (auto& x : v) x = dist(gen);
    return v;
}
std::vector<uint16_t> to_half(const std::vector<float>& v) {
    std::vector<uint16_t> h(v.size());
    for (size_t i = 0; i < v.size(); ++i) h[i] = go_fp32_to_fp16(v[i]);
    return h;
}
std::vector<float> to_float(const std::vector<uint16_t>& h) {
    std::vector<float> v(h.size());
    for (size_t i = 0; i < h.size(); ++i) v[i] = go_fp16_to_fp32(h[i]);
    return v;
}

IComputeBackend* backend() {
    static std::unique_ptr<IComputeBackend> be = [] {
        auto b = create_backend(BackendType::HIP);
        if (b && !b->initialize().ok()) b.reset();
        return b;
    }();
    return be.get();
}

template <typename T>
Tensor upload(std::initializer_list<int64_t> shape, DataType dt, const std::vector<T>& host) {
    auto made = Tensor::allocate(shape, dt, backend());
    if (!made.ok()) return Tensor{};
    Tensor t = made.take();
    if (!backend()->write_buffer(t.buffer(), host.data(), host.size() * sizeof(T)).ok())
        return Tensor{};
    return t;
}
template <typename T>
std::vector<T> download(const Tensor& t) {
    std::vector<T> host(t.size_bytes() / sizeof(T));
    (void)backend()->wait_for_completion();
    (void)backend()->read_buffer(t.buffer(), host.data(), t.size_bytes(), t.buffer_offset());
    return host;
}

}  // namespace

TEST_CASE(backend_buffers) {
    IComputeBackend* be = backend();
    REQUIRE(be != nullptr);
    auto caps = be->get_capabilities();
    CHECK(caps.simd_width == 64 && caps.supports_fp16 && caps.max_buffer_size > (size_t(1) << 30));
    CHECK(caps.name != nullptr && std::strlen(caps.name) > 0);
    CHECK(be->get_type() == BackendType::HIP && be->is_initialized());
    CHECK(is_backend_available(BackendType::HIP) && !is_backend_available(BackendType::Metal));
    CHECK_CODE(be->create_buffer(BufferDesc::device(0)), ErrorCode::InvalidArgument);

    std::vector<uint32_t> pattern(1024);
    for (size_t i = 0; i < pattern.size(); ++i) pattern[i] = uint32_t(i * 2654435761u);
    for (MemoryType kind : {MemoryType::Device, MemoryType::Shared, MemoryType::Managed}) {
        auto made = be->create_buffer({4096, kind, false});
        REQUIRE(made.ok());
        BufferHandle h = made.value();
        CHECK(be->get_native_buffer(h) != nullptr);
        CHECK_OK(be->write_buffer(h, pattern.data(), 4096));
        std::vector<uint32_t> back(1024, 0);
        CHECK_OK(be->read_buffer(h, back.data(), 4096));
        CHECK(back == pattern);
        CHECK_OK(be->read_buffer(h, back.data(), 16, 4080));
        CHECK(back[0] == pattern[1020]);
        CHECK_CODE(be->write_buffer(h, pattern.data(), 4096, 8), ErrorCode::BufferTooSmall);
        CHECK_CODE(be->read_buffer(h, back.data(), 8, 4092), ErrorCode::BufferTooSmall);
        auto mapped = be->map_buffer(h);
        if (kind == MemoryType::Device) {
            CHECK_CODE(mapped, ErrorCode::InvalidArgument);
        } else {
            REQUIRE(mapped.ok());
            auto* p = static_cast<uint32_t*>(mapped.value());
            CHECK(p[5] == pattern[5]);
            p[5] = 0xdeadbeefu;  // host edit, published by unmap
            be->unmap_buffer(h);
            CHECK_OK(be->read_buffer(h, back.data(), 4, 20));
            CHECK(back[0] == 0xdeadbeefu);
        }
        be->destroy_buffer(h);
        CHECK(be->get_native_buffer(h) == nullptr);
    }

    auto a = be->create_buffer_from_host(pattern.data(), BufferDesc::device(4096));
    auto b = be->create_buffer(BufferDesc::managed(4096));
    REQUIRE(a.ok() && b.ok());
    CHECK_OK(be->copy_buffer(a.value(), b.value(), 1024, 1024, 2048));
    CHECK_CODE(be->copy_buffer(a.value(), b.value(), 4096, 1, 0), ErrorCode::BufferTooSmall);
    auto fence = be->create_fence();
    REQUIRE(fence.ok());
    CHECK_OK(be->wait_fence(fence.value()));
    be->destroy_fence(fence.value());
    CHECK_CODE(be->wait_fence(fence.value()), ErrorCode::InvalidArgument);
    std::vector<uint32_t> back(256);
    CHECK_OK(be->read_buffer(b.value(), back.data(), 1024, 2048));
    CHECK(std::memcmp(back.data(), pattern.data() + 256, 1024) == 0);
    CHECK_CODE(be->create_buffer_from_host(nullptr, BufferDesc::device(16)),
               ErrorCode::InvalidArgument);
    CHECK_CODE(be->create_pipeline({}), ErrorCode::NotImplemented);
    CHECK_CODE(be->dispatch(1), ErrorCode::NotImplemented);
    CHECK_OK(be->submit());
    be->destroy_buffer(a.value());
    be->destroy_buffer(b.value());
    CHECK(get_hip_compute() != nullptr && get_hip_compute()->is_initialized());
}

// The reference's attention known-answer test (tests/test_vulkan.cpp:353-482):
// Sq=2, Skv=3, D=4, no mask, Q[i]=i+1, K^T[i]=(i+1)/2, V[i]=(i+1)/4, scale 0.5,
// tolerance 1e-4.  All inputs are exact in binary16.  The tensors go through the registry as
// the reference shapes them ([2, 4] and [3, 4]); the operator pads head size 4 to 64 itself.
// Expected values: tests/golden/vulkan_attention_kat.json.
TEST_CASE(operator_known_answer) {
    REQUIRE(backend() != nullptr);
    const double expected[2][4] = {
        {2.162234681491403, 2.412234681491403, 2.662234681491403, 2.912234681491403},
        {2.248494307269034, 2.498494307269034, 2.748494307269034, 2.998494307269034}};
    // the reference's tensors as they are: Q [2, 4], K and V [3, 4]
    std::vector<float> q(2 * 4), k(3 * 4), v(3 * 4);
    for (int i = 0; i < 2; ++i)
        for (int d = 0; d < 4; ++d) q[i * 4 + d] = float(i * 4 + d + 1);
    for (int d = 0; d < 4; ++d)
        for (int t = 0; t < 3; ++t) k[t * 4 + d] = float(d * 3 + t + 1) * 0.5f;  // K^T is [D, T]
    for (int t = 0; t < 3; ++t)
        for (int d = 0; d < 4; ++d) v[t * 4 + d] = float(t * 4 + d + 1) * 0.25f;

    initialize_operators();
    auto op = OperatorRegistry::instance().create(OpType::ScaledDotProductAttention,
                                                  BackendType::HIP);
    REQUIRE(op != nullptr);
    // all float (the dtypes of tests/test_vulkan.cpp:372-374), float queries over a half cache, all half
    const DataType cases[3][2] = {{DataType::FP32, DataType::FP32}, {DataType::FP32, DataType::FP16},
                                  {DataType::FP16, DataType::FP16}};
    for (const auto& dt : cases) {
        const DataType qdt = dt[0], kvdt = dt[1];
        OpContext ctx;
        ctx.backend = backend();
        Tensor Q = qdt == DataType::FP32 ? upload({2, 4}, qdt, q) : upload({2, 4}, qdt, to_half(q));
        if (kvdt == DataType::FP32)
            ctx.inputs = {Q, upload({3, 4}, kvdt, k), upload({3, 4}, kvdt, v)};
        else
            ctx.inputs = {Q, upload({3, 4}, kvdt, to_half(k)), upload({3, 4}, kvdt, to_half(v))};
        auto shapes = op->infer_shapes(ctx);
        REQUIRE(shapes.ok());
        CHECK((shapes.value()[0] == std::vector<int64_t>{2, 4}));
        auto out = Tensor::allocate(shapes.value()[0], qdt, backend());
        REQUIRE(out.ok());
        ctx.outputs = {out.take()};
        ctx.attrs.set("scale", 0.5);
        ctx.attrs.set("causal", false);
        CHECK_OK(op->validate(ctx));
        CHECK_OK(op->execute(ctx));
        std::vector<float> got = qdt == DataType::FP32 ? download<float>(ctx.outputs[0])
                                                       : to_float(download<uint16_t>(ctx.outputs[0]));
        REQUIRE(got.size() == 8);
        const double tol = qdt == DataType::FP32 ? 1e-4 : 2e-3;  // fp16 output rounding
        for (int i = 0; i < 2; ++i)
            for (int d = 0; d < 4; ++d) CHECK(std::fabs(got[i * 4 + d] - expected[i][d]) <= tol);
        for (auto& t : ctx.inputs) backend()->destroy_buffer(t.buffer());
        backend()->destroy_buffer(ctx.outputs[0].buffer());
    }
}

// A head size with no kernel of its own (80, then 24 and 100): the operator pads to 128 or 64,
// the result must be the oracle's for the unpadded tensors.  Causal, grouped-query, start_pos > 0.
TEST_CASE(operator_other_head_sizes_vs_oracle) {
    REQUIRE(backend() != nullptr);
    initialize_operators();
    auto op = OperatorRegistry::instance().create(OpType::ScaledDotProductAttention, BackendType::HIP);
    REQUIRE(op != nullptr);
    for (int dim : {80, 24, 100}) {
        const int H = 4, Hkv = 2, seq_q = 19, seq_kv = 50, start = seq_kv - seq_q;
        auto q = randn(size_t(H) * seq_q * dim, 600 + dim);                 // [H, seq_q, dim]
        auto kh = to_half(randn(size_t(Hkv) * seq_kv * dim, 601 + dim));    // [Hkv, seq_kv, dim]
        auto vh = to_half(randn(size_t(Hkv) * seq_kv * dim, 602 + dim));
        OpContext ctx;
        ctx.backend = backend();
        ctx.inputs = {upload({H, seq_q, dim}, DataType::FP32, q), upload({Hkv, seq_kv, dim}, DataType::FP16, kh),
                      upload({Hkv, seq_kv, dim}, DataType::FP16, vh)};
        auto out = Tensor::allocate({H, seq_q, dim}, DataType::FP32, backend());
        REQUIRE(out.ok());
        ctx.outputs = {out.take()};
        ctx.attrs.set("start_pos", int64_t(start));
        CHECK_OK(op->execute(ctx));
        auto got = download<float>(ctx.outputs[0]);
        // oracle layouts: q [seq_q, H, dim], cache [Hkv, max_seq, dim] halves, out [seq_q, H * dim]
        std::vector<float> q_tok(q.size()), want_tok(q.size()), want(q.size());
        for (int h = 0; h < H; ++h)
            for (int s = 0; s < seq_q; ++s)
                std::memcpy(&q_tok[(size_t(s) * H + h) * dim], &q[(size_t(h) * seq_q + s) * dim], dim * 4);
        go_attention_cached(q_tok.data(), kh.data(), vh.data(), want_tok.data(), nullptr, 1, seq_q, H, Hkv, dim,
                            seq_kv, seq_kv, start, 1.0f / std::sqrt(float(dim)));
        for (int h = 0; h < H; ++h)
            for (int s = 0; s < seq_q; ++s)
                std::memcpy(&want[(size_t(h) * seq_q + s) * dim], &want_tok[(size_t(s) * H + h) * dim], dim * 4);
        CHECK(close_enough(got, want, "operator, head size without a kernel"));
        for (auto& t : ctx.inputs) backend()->destroy_buffer(t.buffer());
        backend()->destroy_buffer(ctx.outputs[0].buffer());
    }
    // float K and V (what the reference's operator tests allocate): a head size with a kernel and
    // one without, several batch entries; the values are halves widened to float, so that the
    // oracle's half cache holds exactly what the operator's conversion produces
    for (int dim : {128, 40}) {
        const int B = 2, H = 4, Hkv = 2, seq_q = 21, seq_kv = 37, start = seq_kv - seq_q;
        auto q = randn(size_t(B) * H * seq_q * dim, 700 + dim);                     // [B, H, seq_q, dim]
        auto kh = to_half(randn(size_t(B) * Hkv * seq_kv * dim, 701 + dim));        // [B, Hkv, seq_kv, dim]
        auto vh = to_half(randn(size_t(B) * Hkv * seq_kv * dim, 702 + dim));
        OpContext ctx;
        ctx.backend = backend();
        ctx.inputs = {upload({B, H, seq_q, dim}, DataType::FP32, q),
                      upload({B, Hkv, seq_kv, dim}, DataType::FP32, to_float(kh)),
                      upload({B, Hkv, seq_kv, dim}, DataType::FP32, to_float(vh))};
        auto out = Tensor::allocate({B, H, seq_q, dim}, DataType::FP32, backend());
        REQUIRE(out.ok());
        ctx.outputs = {out.take()};
        ctx.attrs.set("start_pos", int64_t(start));
        CHECK_OK(op->execute(ctx));
        auto got = download<float>(ctx.outputs[0]);
        std::vector<float> want(q.size());
        for (int b = 0; b < B; ++b) {
            const size_t qo = size_t(b) * H * seq_q * dim, ko = size_t(b) * Hkv * seq_kv * dim;
            std::vector<float> q_tok(size_t(H) * seq_q * dim), want_tok(q_tok.size());
            for (int h = 0; h < H; ++h)
                for (int s = 0; s < seq_q; ++s)
                    std::memcpy(&q_tok[(size_t(s) * H + h) * dim], &q[qo + (size_t(h) * seq_q + s) * dim], dim * 4);
            go_attention_cached(q_tok.data(), kh.data() + ko, vh.data() + ko, want_tok.data(), nullptr, 1, seq_q, H,
                                Hkv, dim, seq_kv, seq_kv, start, 1.0f / std::sqrt(float(dim)));
            for (int h = 0; h < H; ++h)
                for (int s = 0; s < seq_q; ++s)
                    std::memcpy(&want[qo + (size_t(h) * seq_q + s) * dim], &want_tok[(size_t(s) * H + h) * dim],
                                dim * 4);
        }
        CHECK(close_enough(got, want, "operator, float K and V"));
        for (auto& t : ctx.inputs) backend()->destroy_buffer(t.buffer());
        backend()->destroy_buffer(ctx.outputs[0].buffer());
    }
    // beyond 128 there is nothing to pad to
    OpContext big;
    big.backend = backend();
    big.inputs = {upload({2, 160}, DataType::FP32, randn(320, 1)), upload({3, 160}, DataType::FP16, to_half(randn(480, 2))),
                  upload({3, 160}, DataType::FP16, to_half(randn(480, 3)))};
    CHECK_CODE(op->validate(big), ErrorCode::NotImplemented);
    for (auto& t : big.inputs) backend()->destroy_buffer(t.buffer());
}

// Causal, grouped-query, chunk at start_pos > 0 through the operator, against
// the oracle's cached attention (transformer.mm:1703-1840 restated).
TEST_CASE(operator_causal_gqa_vs_oracle) {
    REQUIRE(backend() != nullptr);
    const int H = 8, Hkv = 2, Sq = 96, start = 37, Skv = start + Sq;
    auto q = randn(size_t(H) * Sq * D, 11);                 // [H, Sq, D]
    auto kh = to_half(randn(size_t(Hkv) * Skv * D, 12));    // [Hkv, Skv, D]
    auto vh = to_half(randn(size_t(Hkv) * Skv * D, 13));
    auto op = OperatorRegistry::instance().create(OpType::ScaledDotProductAttention,
                                                  BackendType::HIP);
    REQUIRE(op != nullptr);
    OpContext ctx;
    ctx.backend = backend();
    ctx.inputs = {upload({H, Sq, D}, DataType::FP32, q), upload({Hkv, Skv, D}, DataType::FP16, kh),
                  upload({Hkv, Skv, D}, DataType::FP16, vh)};
    ctx.outputs = {Tensor::allocate({H, Sq, D}, DataType::FP32, backend()).take()};
    ctx.attrs.set("start_pos", int64_t(start));
    CHECK_OK(op->execute(ctx));  // scale defaults to 1/sqrt(D)
    auto got = download<float>(ctx.outputs[0]);

    std::vector<float> q_tok(q.size()), want_tok(q.size()), want(q.size());
    for (int h = 0; h < H; ++h)
        for (int s = 0; s < Sq; ++s)
            std::memcpy(&q_tok[(size_t(s) * H + h) * D], &q[(size_t(h) * Sq + s) * D], D * 4);
    go_attention_cached(q_tok.data(), kh.data(), vh.data(), want_tok.data(), nullptr, 1, Sq, H, Hkv,
                        D, Skv, Skv, start, 1.0f / std::sqrt(float(D)));
    for (int h = 0; h < H; ++h)
        for (int s = 0; s < Sq; ++s)
            std::memcpy(&want[(size_t(h) * Sq + s) * D], &want_tok[(size_t(s) * H + h) * D], D * 4);
    CHECK(close_enough(got, want, "operator causal GQA"));
    for (auto& t : ctx.inputs) backend()->destroy_buffer(t.buffer());
    backend()->destroy_buffer(ctx.outputs[0].buffer());
}

TEST_CASE(kv_cache_append_on_device) {
    REQUIRE(backend() != nullptr);
    ModelConfig cfg;
    cfg.num_layers = 2;
    cfg.num_kv_heads = 2;
    cfg.num_heads = 4;
    cfg.head_dim = D;
    const int max_seq = 64;
    auto made = KVCache::allocate(cfg, max_seq, backend());
    REQUIRE(made.ok());
    KVCache cache = made.take();
    const size_t cache_elems = size_t(cfg.num_kv_heads) * max_seq * D;
    // the oracle appends into caches that start from the same bytes as the device's
    std::vector<std::vector<uint16_t>> want_k, want_v;
    for (int l = 0; l < 2; ++l) {
        want_k.push_back(download<uint16_t>(cache.get(l).first));
        want_v.push_back(download<uint16_t>(cache.get(l).second));
    }
    int len = 0;
    uint32_t seed = 100;
    for (int new_len : {5, 1, 26}) {
        for (int l = 0; l < 2; ++l) {
            auto kh = to_half(randn(size_t(2) * new_len * D, seed++));
            auto vh = to_half(randn(size_t(2) * new_len * D, seed++));
            Tensor nk = upload({1, 2, new_len, D}, DataType::FP16, kh);
            Tensor nv = upload({1, 2, new_len, D}, DataType::FP16, vh);
            CHECK_OK(cache.append(l, nk, nv));
            CHECK(cache.seq_len() == (l == 1 ? len + new_len : len));  // advances on the last layer
            CHECK(go_kv_cache_append_f16(want_k[l].data(), kh.data(), 2, D, len, new_len, max_seq) == 0);
            CHECK(go_kv_cache_append_f16(want_v[l].data(), vh.data(), 2, D, len, new_len, max_seq) == 0);
            (void)backend()->wait_for_completion();
            backend()->destroy_buffer(nk.buffer());
            backend()->destroy_buffer(nv.buffer());
        }
        len += new_len;
    }
    CHECK(cache.seq_len() == 32);
    for (int l = 0; l < 2; ++l) {
        CHECK(download<uint16_t>(cache.get(l).first) == want_k[l]);   // bit exact
        CHECK(download<uint16_t>(cache.get(l).second) == want_v[l]);
        CHECK(want_k[l].size() == cache_elems);
    }
    Tensor big = upload({1, 2, 33, D}, DataType::FP16, std::vector<uint16_t>(size_t(2) * 33 * D, 0));
    CHECK_CODE(cache.append(0, big, big), ErrorCode::InvalidArgument);  // 32 + 33 > 64
    CHECK(cache.seq_len() == 32);
    cache.truncate(10);
    CHECK(cache.seq_len() == 10);

    // Attention over what the cache holds: decode one token against 10 cached rows.
    auto q = randn(size_t(4) * D, 77);
    Tensor Q = upload({4, 1, D}, DataType::FP32, q);
    Tensor out = Tensor::allocate({4, 1, D}, DataType::FP32, backend()).take();
    HipCompute* hc = get_hip_compute();
    REQUIRE(hc != nullptr);
    auto [ck, cv] = cache.get(1);
    CHECK_OK(hc->multihead_attention(hip_device_pointer(backend(), Q.buffer()),
                                     hip_device_pointer(backend(), ck.buffer()),
                                     hip_device_pointer(backend(), cv.buffer()),
                                     hip_device_pointer(backend(), out.buffer()), 4, 2, 1, 10, D,
                                     0.09f, max_seq));
    hc->sync();
    std::vector<float> want(q.size());
    go_attention_cached(q.data(), want_k[1].data(), want_v[1].data(), want.data(), nullptr, 1, 1, 4,
                        2, D, 10, max_seq, 9, 0.09f);
    CHECK(close_enough(download<float>(out), want, "decode over KVCache"));
}

TEST_CASE(paged_pool_append_and_batched_decode) {
    REQUIRE(backend() != nullptr);
    HipCompute* hc = get_hip_compute();
    REQUIRE(hc != nullptr);
    ModelConfig cfg;
    cfg.num_layers = 1;
    cfg.num_kv_heads = 2;
    cfg.num_heads = 8;
    cfg.head_dim = D;
    const int bs = 16, batch = 3;
    const int lens[batch] = {40, 17, 100};
    PagedKVPool pool;
    CHECK_OK(pool.initialize(cfg, batch, 256, bs, backend()));
    BlockManager& mgr = pool.block_manager();
    const size_t pool_elems = size_t(mgr.num_total_blocks()) * bs * 2 * D;
    auto want_k = download<uint16_t>(mgr.k_cache(0));
    auto want_v = download<uint16_t>(mgr.v_cache(0));
    CHECK(want_k.size() == pool_elems);
    void* k_pool = hip_device_pointer(backend(), mgr.k_cache(0).buffer());
    void* v_pool = hip_device_pointer(backend(), mgr.v_cache(0).buffer());

    // interleave the sequences' growth so that their blocks interleave too
    int slots[batch];
    for (int b = 0; b < batch; ++b) slots[b] = pool.acquire_slot();
    uint32_t seed = 500;
    int done[batch] = {0, 0, 0};
    for (int round = 0; round < 7; ++round)
        for (int b = 0; b < batch; ++b) {
            const int step = std::min(lens[b] - done[b], b == 2 ? 15 : 9);
            if (step <= 0) continue;
            PagedKVCache& seq = pool.get_cache(slots[b]);
            REQUIRE(seq.append_tokens(step));
            auto nk = randn(size_t(2) * step * D, seed++);  // [Hkv, step, D] float
            auto nv = randn(size_t(2) * step * D, seed++);
            std::vector<int32_t> table(seq.block_table().begin(), seq.block_table().end());
            HipBuffer* d_k = hc->create_buffer(nk.size() * 4);
            HipBuffer* d_v = hc->create_buffer(nv.size() * 4);
            HipBuffer* d_t = hc->create_buffer(table.size() * 4);
            REQUIRE(d_k && d_v && d_t);
            CHECK_OK(hc->upload(d_k, nk.data(), nk.size() * 4));
            CHECK_OK(hc->upload(d_v, nv.data(), nv.size() * 4));
            CHECK_OK(hc->upload(d_t, table.data(), table.size() * 4));
            CHECK_OK(hc->paged_kv_cache_append(d_k, d_v, k_pool, v_pool, d_t, 2, D, done[b], step, bs));
            hc->sync();
            go_paged_kv_cache_append_f32(want_k.data(), nk.data(), table.data(), 2, D, done[b], step, bs);
            go_paged_kv_cache_append_f32(want_v.data(), nv.data(), table.data(), 2, D, done[b], step, bs);
            hc->release_buffer(d_k);
            hc->release_buffer(d_v);
            hc->release_buffer(d_t);
            done[b] += step;
        }
    for (int b = 0; b < batch; ++b) CHECK(pool.get_cache(slots[b]).seq_len() == lens[b]);
    CHECK(download<uint16_t>(mgr.k_cache(0)) == want_k);  // bit exact
    CHECK(download<uint16_t>(mgr.v_cache(0)) == want_v);

    const int max_blocks = 8;
    std::vector<int32_t> tables(size_t(batch) * max_blocks, 0), seq_lens(lens, lens + batch);
    for (int b = 0; b < batch; ++b) {
        const auto& t = pool.get_cache(slots[b]).block_table();
        std::copy(t.begin(), t.end(), tables.begin() + size_t(b) * max_blocks);
    }
    auto q = randn(size_t(batch) * 8 * D, 900);
    HipBuffer* d_q = hc->create_buffer(q.size() * 4);
    HipBuffer* d_o = hc->create_buffer(q.size() * 4);
    HipBuffer* d_t = hc->create_buffer(tables.size() * 4);
    HipBuffer* d_l = hc->create_buffer(seq_lens.size() * 4);
    REQUIRE(d_q && d_o && d_t && d_l);
    CHECK_OK(hc->upload(d_q, q.data(), q.size() * 4));
    CHECK_OK(hc->upload(d_t, tables.data(), tables.size() * 4));
    CHECK_OK(hc->upload(d_l, seq_lens.data(), seq_lens.size() * 4));
    const float scale = 1.0f / std::sqrt(float(D));
    CHECK_OK(hc->batched_paged_attention_decode(d_q, k_pool, v_pool, d_t, d_l, d_o, batch, 8, 2, D,
                                                bs, max_blocks, scale));
    std::vector<float> got(q.size()), want(q.size());
    CHECK_OK(hc->download(got.data(), d_o, got.size() * 4));
    go_batched_paged_decode(q.data(), want_k.data(), want_v.data(), tables.data(), seq_lens.data(),
                            want.data(), nullptr, batch, 8, 2, D, bs, max_blocks, scale);
    CHECK(close_enough(got, want, "batched paged decode"));

    // single-sequence entry point on the longest sequence
    std::vector<float> got1(size_t(8) * D), want1(want.begin() + size_t(2) * 8 * D, want.end());
    CHECK_OK(hc->paged_attention_decode(static_cast<char*>(d_q) + size_t(2) * 8 * D * 4, k_pool, v_pool,
                                        static_cast<char*>(d_t) + size_t(2) * max_blocks * 4, d_o, 8, 2,
                                        lens[2], D, bs, scale));
    CHECK_OK(hc->download(got1.data(), d_o, got1.size() * 4));
    CHECK(close_enough(got1, want1, "paged decode, one sequence"));
    for (HipBuffer* p : {d_q, d_o, d_t, d_l}) hc->release_buffer(p);
    for (int b = 0; b < batch; ++b) pool.release_slot(slots[b]);
    CHECK(pool.num_free_blocks() == mgr.num_total_blocks());
}

TEST_CASE(speculation_tree_attention) {
    REQUIRE(backend() != nullptr);
    HipCompute* hc = get_hip_compute();
    REQUIRE(hc != nullptr);
    SpeculationTree tree;
    tree.add_node(1, -1);
    std::mt19937 gen(4242);
    for (int i = 1; i < 23; ++i) tree.add_node(i + 1, int(gen() % uint32_t(i)));
    const std::vector<int> parents_int = tree.get_parent_indices();
    std::vector<int32_t> parents(parents_int.begin(), parents_int.end());
    const int N = int(tree.size()), H = 4, Hkv = 2, cache_len = 75;
    auto q = randn(size_t(H) * N * D, 31);                       // [H, N, D]
    auto ck = to_half(randn(size_t(Hkv) * cache_len * D, 32));   // [Hkv, cache_len, D]
    auto cv = to_half(randn(size_t(Hkv) * cache_len * D, 33));
    auto tk = to_half(randn(size_t(Hkv) * N * D, 34));           // [Hkv, N, D]
    auto tv = to_half(randn(size_t(Hkv) * N * D, 35));
    const float scale = 0.1f;

    auto dev = [&](const void* p, size_t bytes) {
        HipBuffer* d = hc->create_buffer(bytes);
        if (d) (void)hc->upload(d, p, bytes);
        return d;
    };
    HipBuffer* d_q = dev(q.data(), q.size() * 4);
    HipBuffer* d_ck = dev(ck.data(), ck.size() * 2);
    HipBuffer* d_cv = dev(cv.data(), cv.size() * 2);
    HipBuffer* d_tk = dev(tk.data(), tk.size() * 2);
    HipBuffer* d_tv = dev(tv.data(), tv.size() * 2);
    HipBuffer* d_p = dev(parents.data(), parents.size() * 4);
    HipBuffer* d_o = hc->create_buffer(q.size() * 4);
    REQUIRE(d_q && d_ck && d_cv && d_tk && d_tv && d_p && d_o);
    CHECK_OK(hc->attention_tree(d_q, d_ck, d_cv, d_tk, d_tv, d_p, d_o, H, Hkv, N, cache_len, D, scale));
    std::vector<float> got(q.size());
    CHECK_OK(hc->download(got.data(), d_o, got.size() * 4));

    // oracle layouts: q [N, H, D], tree K/V [N, Hkv, D] floats, output [N, H*D]
    std::vector<float> q_tok(q.size()), tkf(tk.size()), tvf(tv.size()), want_tok(q.size()),
        want(q.size());
    auto tk32 = to_float(tk), tv32 = to_float(tv);
    for (int h = 0; h < H; ++h)
        for (int n = 0; n < N; ++n)
            std::memcpy(&q_tok[(size_t(n) * H + h) * D], &q[(size_t(h) * N + n) * D], D * 4);
    for (int h = 0; h < Hkv; ++h)
        for (int n = 0; n < N; ++n) {
            std::memcpy(&tkf[(size_t(n) * Hkv + h) * D], &tk32[(size_t(h) * N + n) * D], D * 4);
            std::memcpy(&tvf[(size_t(n) * Hkv + h) * D], &tv32[(size_t(h) * N + n) * D], D * 4);
        }
    CHECK(go_attention_tree(q_tok.data(), ck.data(), cv.data(), nullptr, 0, cache_len, tkf.data(),
                            tvf.data(), parents.data(), want_tok.data(), nullptr, 1, N, H, Hkv, D,
                            cache_len, scale) == 0);
    for (int h = 0; h < H; ++h)
        for (int n = 0; n < N; ++n)
            std::memcpy(&want[(size_t(h) * N + n) * D], &want_tok[(size_t(n) * H + h) * D], D * 4);
    CHECK(close_enough(got, want, "tree attention over SpeculationTree parents"));
    for (HipBuffer* p : {d_q, d_ck, d_cv, d_tk, d_tv, d_p, d_o}) hc->release_buffer(p);
}

// float -> half, round to nearest even (what the GPU path's conversion does)
uint16_t half_nearest(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
    x &= 0x7FFFFFFFu;
    if (x > 0x7F800000u) return sign | 0x7E00u;
    if (x >= 0x477FF000u) return sign | 0x7C00u;  // 65520 and above round to infinity
    if (x < 0x38800000u) {                         // below the smallest normal half
        if (x < 0x33000000u) return sign;          // at most half of the smallest subnormal
        const int shift = 126 - static_cast<int>(x >> 23);
        const uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
        uint32_t h = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) ++h;
        return sign | static_cast<uint16_t>(h);
    }
    uint32_t h = (x - 0x38000000u) >> 13;
    const uint32_t rem = x & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
    return sign | static_cast<uint16_t>(h);
}

TEST_CASE(rope_cache_apply_and_append) {
    REQUIRE(backend() != nullptr);
    const int max_pos = 300, hq = 6, hkv = 2, seq = 21, start = 250;
    RoPECache rope;
    Tensor dummy = Tensor::allocate({1, 1, 1, D}, DataType::FP32, backend()).take();
    CHECK_CODE(rope.apply(dummy, dummy, 0, backend()), ErrorCode::InvalidState);  // rope.cpp:25-27
    rope.initialize(max_pos, D, 10000.0f);
    REQUIRE(rope.is_initialized());
    // the host tables are the reference's (and the oracle's) to the bit
    std::vector<float> cos_t(size_t(max_pos) * D / 2), sin_t(cos_t.size());
    go_rope_table(cos_t.data(), sin_t.data(), max_pos, D, 10000.0f);
    CHECK(rope.cos_cache() == cos_t);
    CHECK(rope.sin_cache() == sin_t);

    auto q = randn(size_t(seq) * hq * D, 901), k = randn(size_t(seq) * hkv * D, 902),
         v = randn(size_t(seq) * hkv * D, 903);
    Tensor Q = upload({1, seq, hq, D}, DataType::FP32, q);
    Tensor K = upload({1, seq, hkv, D}, DataType::FP32, k);
    Tensor V = upload({1, seq, hkv, D}, DataType::FP32, v);
    CHECK_OK(rope.apply(Q, K, start, backend()));
    auto want_q = q, want_k = k;
    CHECK(go_rope_apply(want_q.data(), seq, hq, D, start, cos_t.data(), sin_t.data(), max_pos) == 0);
    CHECK(go_rope_apply(want_k.data(), seq, hkv, D, start, cos_t.data(), sin_t.data(), max_pos) == 0);
    CHECK(download<float>(Q) == want_q);  // bit exact
    CHECK(download<float>(K) == want_k);
    // the range check of rope.cpp:34-38
    CHECK_CODE(rope.apply(Q, K, max_pos - seq + 1, backend()), ErrorCode::InvalidArgument);

    // rotate and append in one pass: cache rows are the rounded rotated K and V
    const int max_len = 280;
    Tensor K2 = upload({1, seq, hkv, D}, DataType::FP32, k);
    Tensor Q2 = upload({1, seq, hq, D}, DataType::FP32, q);
    std::vector<uint16_t> sentinel(size_t(hkv) * max_len * D, 0x1234);
    Tensor CK = upload({hkv, max_len, D}, DataType::FP16, sentinel);
    Tensor CV = upload({hkv, max_len, D}, DataType::FP16, sentinel);
    CHECK_OK(rope.apply_and_append(Q2, K2, V, CK, CV, start, backend()));
    CHECK(download<float>(Q2) == want_q);
    auto got_k = download<uint16_t>(CK), got_v = download<uint16_t>(CV);
    size_t wrong = 0;
    for (int h = 0; h < hkv; ++h)
        for (int pos = 0; pos < max_len; ++pos)
            for (int d = 0; d < D; ++d) {
                const size_t at = (size_t(h) * max_len + pos) * D + d;
                uint16_t wk = 0x1234, wv = 0x1234;
                if (pos >= start && pos < start + seq) {
                    const size_t src = (size_t(pos - start) * hkv + h) * D + d;
                    wk = half_nearest(want_k[src]);
                    wv = half_nearest(v[src]);
                }
                wrong += (got_k[at] != wk) + (got_v[at] != wv);
            }
    CHECK(wrong == 0);
    CHECK_CODE(rope.apply_and_append(Q2, K2, V, CK, CV, 270, backend()), ErrorCode::InvalidArgument);
}

TEST_CASE(paged_prefill_then_batched_decode_steps) {
    REQUIRE(backend() != nullptr);
    HipCompute* hc = get_hip_compute();
    REQUIRE(hc != nullptr);
    ModelConfig cfg;
    cfg.num_layers = 2;
    cfg.num_heads = 8;
    cfg.num_kv_heads = 2;
    cfg.head_dim = D;
    const int bs = 16, hq = 8, hkv = 2, max_blocks = 12, max_pos = max_blocks * bs;
    PagedKVPool pool;
    REQUIRE(pool.initialize(cfg, 5, 26 * bs, bs, backend()).ok());  // 26 blocks in all
    BlockManager& mgr = pool.block_manager();
    RoPECache rope;
    rope.initialize(max_pos, D, 10000.0f);
    std::vector<float> cos_t(size_t(max_pos) * D / 2), sin_t(cos_t.size());
    go_rope_table(cos_t.data(), sin_t.data(), max_pos, D, 10000.0f);
    auto rope_tables = rope.device_tables(backend());
    REQUIRE(rope_tables.ok());
    const float scale = 1.0f / std::sqrt(float(D));

    // the oracle's pools start from the device's bytes
    std::vector<std::vector<uint16_t>> want_k, want_v;
    for (int l = 0; l < 2; ++l) {
        want_k.push_back(download<uint16_t>(mgr.k_cache(l)));
        want_v.push_back(download<uint16_t>(mgr.v_cache(l)));
    }

    // ---- paged prefill: every sequence's prompt in one rotate-and-append launch per layer
    // (the reference fills a paged cache one token at a time,
    // tools/benchmark_paged_attention.mm:348-363)
    const int batch = 4;
    const int prompt[batch] = {37, 1, 150, 64};
    int slots[batch];
    uint32_t seed = 7000;
    for (int b = 0; b < batch; ++b) {
        slots[b] = pool.acquire_slot();
        REQUIRE(slots[b] >= 0);
        PagedKVCache& seq = pool.get_cache(slots[b]);
        REQUIRE(seq.append_tokens(prompt[b]));
        std::vector<int32_t> table(seq.block_table().begin(), seq.block_table().end());
        Tensor T = upload({int64_t(table.size())}, DataType::INT32, table);
        for (int l = 0; l < 2; ++l) {
            auto k = randn(size_t(prompt[b]) * hkv * D, seed++), v = randn(size_t(prompt[b]) * hkv * D, seed++);
            Tensor K = upload({prompt[b], hkv, D}, DataType::FP32, k);
            Tensor V = upload({prompt[b], hkv, D}, DataType::FP32, v);
            granite_hip_rope_args r{};
            r.k = hip_device_pointer(backend(), K.buffer());
            r.v = hip_device_pointer(backend(), V.buffer());
            r.cache_k = hip_device_pointer(backend(), mgr.k_cache(l).buffer());
            r.cache_v = hip_device_pointer(backend(), mgr.v_cache(l).buffer());
            r.block_table = static_cast<const int32_t*>(hip_device_pointer(backend(), T.buffer()));
            r.block_size = bs;
            r.num_heads_k = hkv;
            r.seq_len = uint32_t(prompt[b]);
            r.head_dim = D;
            r.start_pos = 0;
            r.cos_table = rope_tables.value().first;
            r.sin_table = rope_tables.value().second;
            r.table_positions = max_pos;
            r.rounding = GRANITE_HIP_ROUND_TRUNCATE;
            CHECK_OK(hc->rope_append(r));
            hc->sync();
            // oracle: rotate, then the paged append on [Hkv, new_len, D]
            CHECK(go_rope_apply(k.data(), prompt[b], hkv, D, 0, cos_t.data(), sin_t.data(), max_pos) == 0);
            std::vector<float> kt(k.size()), vt(v.size());
            for (int s = 0; s < prompt[b]; ++s)
                for (int h = 0; h < hkv; ++h)
                    for (int d = 0; d < D; ++d) {
                        kt[(size_t(h) * prompt[b] + s) * D + d] = k[(size_t(s) * hkv + h) * D + d];
                        vt[(size_t(h) * prompt[b] + s) * D + d] = v[(size_t(s) * hkv + h) * D + d];
                    }
            go_paged_kv_cache_append_f32(want_k[l].data(), kt.data(), table.data(), hkv, D, 0, prompt[b], bs);
            go_paged_kv_cache_append_f32(want_v[l].data(), vt.data(), table.data(), hkv, D, 0, prompt[b], bs);
            backend()->destroy_buffer(K.buffer());
            backend()->destroy_buffer(V.buffer());
        }
        backend()->destroy_buffer(T.buffer());
    }
    for (int l = 0; l < 2; ++l) {
        CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);  // bit exact
        CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
    }

    // ---- batched decode steps
    PagedDecodeBatch step;
    CHECK_CODE(step.begin_step(std::span<const int>(slots, batch)), ErrorCode::InvalidState);
    REQUIRE(step.initialize(&pool, 8, max_blocks, backend()).ok());
    step.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
    Tensor Qbad = Tensor::allocate({batch, hq, D}, DataType::FP32, backend()).take();
    CHECK_CODE(step.run_layer(0, Qbad, Qbad, Qbad, Qbad, scale, &rope), ErrorCode::InvalidState);
    int lens[batch];
    for (int b = 0; b < batch; ++b) lens[b] = prompt[b];
    for (int it = 0; it < 3; ++it) {
        auto failed = step.begin_step(std::span<const int>(slots, batch));
        REQUIRE(failed.ok());
        CHECK(failed.value().empty());
        CHECK(step.batch_size() == batch);
        std::vector<int32_t> tables(size_t(batch) * max_blocks, 0), seq_lens(batch);
        for (int b = 0; b < batch; ++b) {
            lens[b] += 1;
            CHECK(pool.get_cache(slots[b]).seq_len() == lens[b]);
            CHECK(step.seq_lens()[b] == lens[b]);
            seq_lens[b] = lens[b];
            const auto& t = pool.get_cache(slots[b]).block_table();
            std::copy(t.begin(), t.end(), tables.begin() + size_t(b) * max_blocks);
        }
        for (int l = 0; l < 2; ++l) {
            auto q = randn(size_t(batch) * hq * D, seed++), k = randn(size_t(batch) * hkv * D, seed++),
                 v = randn(size_t(batch) * hkv * D, seed++);
            Tensor Q = upload({batch, hq, D}, DataType::FP32, q);
            Tensor K = upload({batch, hkv, D}, DataType::FP32, k);
            Tensor V = upload({batch, hkv, D}, DataType::FP32, v);
            Tensor O = Tensor::allocate({batch, hq, D}, DataType::FP32, backend()).take();
            CHECK_OK(step.run_layer(l, Q, K, V, O, scale, &rope));
            // oracle: sequence by sequence, as the reference's loop would
            for (int b = 0; b < batch; ++b) {
                const int pos = lens[b] - 1;
                CHECK(go_rope_apply(q.data() + size_t(b) * hq * D, 1, hq, D, pos, cos_t.data(), sin_t.data(), max_pos) == 0);
                CHECK(go_rope_apply(k.data() + size_t(b) * hkv * D, 1, hkv, D, pos, cos_t.data(), sin_t.data(), max_pos) == 0);
                go_paged_kv_cache_append_f32(want_k[l].data(), k.data() + size_t(b) * hkv * D,
                                             tables.data() + size_t(b) * max_blocks, hkv, D, pos, 1, bs);
                go_paged_kv_cache_append_f32(want_v[l].data(), v.data() + size_t(b) * hkv * D,
                                             tables.data() + size_t(b) * max_blocks, hkv, D, pos, 1, bs);
            }
            std::vector<float> want(q.size());
            go_batched_paged_decode(q.data(), want_k[l].data(), want_v[l].data(), tables.data(), seq_lens.data(),
                                    want.data(), nullptr, batch, hq, hkv, D, bs, max_blocks, scale);
            CHECK(download<float>(Q) == q);                           // rotated Q and K: the oracle's bits
            CHECK(download<float>(K) == k);
            CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);   // pools bit exact
            CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
            CHECK(close_enough(download<float>(O), want, "batched decode step"));
            for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
        }
    }

    // ---- a sequence that cannot take a token: reported, left out, the others go on
    // 37+3, 1+3, 150+3, 64+3 tokens hold 3 + 1 + 10 + 5 = 19 of 26 blocks; a fifth sequence takes the rest
    int extra = pool.acquire_slot();
    REQUIRE(extra >= 0);
    REQUIRE(pool.get_cache(extra).append_tokens(7 * bs));
    CHECK(pool.num_free_blocks() == 0);
    // sequence 3 is at 67 tokens: 5 blocks hold 80, so it still fits; sequence 2 at 153 of 160 too;
    // push sequence 0 (40 tokens, 3 blocks = 48) to its block edge to make it need a new block
    REQUIRE(pool.get_cache(slots[0]).append_tokens(8));
    lens[0] += 8;
    {
        auto failed = step.begin_step(std::span<const int>(slots, batch));
        REQUIRE(failed.ok());
        REQUIRE(failed.value().size() == 1);
        CHECK(failed.value()[0] == slots[0]);
        CHECK(step.seq_lens()[0] == 0);
        CHECK(pool.get_cache(slots[0]).seq_len() == lens[0]);  // unchanged
        auto q = randn(size_t(batch) * hq * D, seed++), k = randn(size_t(batch) * hkv * D, seed++),
             v = randn(size_t(batch) * hkv * D, seed++);
        Tensor Q = upload({batch, hq, D}, DataType::FP32, q);
        Tensor K = upload({batch, hkv, D}, DataType::FP32, k);
        Tensor V = upload({batch, hkv, D}, DataType::FP32, v);
        std::vector<float> sentinel(q.size(), -7.0f);
        Tensor O = upload({batch, hq, D}, DataType::FP32, sentinel);
        CHECK_OK(step.run_layer(0, Q, K, V, O, scale, &rope));
        auto got_q = download<float>(Q), got_o = download<float>(O);
        bool untouched = true;
        for (size_t i = 0; i < size_t(hq) * D; ++i) untouched = untouched && got_q[i] == q[i] && got_o[i] == -7.0f;
        CHECK(untouched);                                  // row 0: neither rotated nor written
        bool others_written = true;
        for (size_t i = size_t(hq) * D; i < got_o.size(); ++i) others_written = others_written && got_o[i] != -7.0f;
        CHECK(others_written);
        CHECK(download<uint16_t>(mgr.k_cache(1)) == want_k[1]);  // the other layer's pool is not touched
    }
    CHECK_CODE(step.begin_step(std::span<const int>(slots, 0)), ErrorCode::InvalidArgument);
}

// The chunk loop of forward_prefill_raw (src/llm/transformer.mm:3467-3477, 3681-3866) on the
// host layer: a 2048-token prompt fed in chunks of 512 and of 96 (ragged last chunk), then a
// second prompt behind it in chunks of 128, into a paged sequence; and a prompt into a
// contiguous KVCache.  Every chunk's rotated Q/K, the caches and the outputs are compared
// with the oracle's one-shot pass over the whole prompt: rotation and cache rows bit for bit
// (truncating conversion), outputs within the attention tolerance.
TEST_CASE(chunked_prefill_driver) {
    REQUIRE(backend() != nullptr);
    CHECK(prefill_chunk_tokens(2048, 0) == 2048);       // no chunking asked for
    CHECK(prefill_chunk_tokens(2048, 4096) == 2048);    // chunk not below the prompt
    CHECK(prefill_chunk_tokens(2048, 512) == 512);
    CHECK(prefill_chunk_tokens(2048, 7) == 32);         // raised to the minimum of 32
    CHECK(prefill_chunk_tokens(20, 7) == 20);           // 32 capped by the prompt
    const int hq = 8, hkv = 2, bs = 16, layers = 2;
    const int max_pos = 2560;
    const float scale = 1.0f / std::sqrt(float(D));
    RoPECache rope;
    rope.initialize(max_pos, D, 10000.0f);
    std::vector<float> cos_t(size_t(max_pos) * D / 2), sin_t(cos_t.size());
    go_rope_table(cos_t.data(), sin_t.data(), max_pos, D, 10000.0f);

    auto transpose_heads = [&](const std::vector<float>& x, int n) {  // [n, hkv, D] -> [hkv, n, D]
        std::vector<float> t(x.size());
        for (int s = 0; s < n; ++s)
            for (int h = 0; h < hkv; ++h)
                std::memcpy(&t[(size_t(h) * n + s) * D], &x[(size_t(s) * hkv + h) * D], D * sizeof(float));
        return t;
    };

    // ---- paged sequence
    ModelConfig cfg;
    cfg.num_layers = layers;
    cfg.num_heads = hq;
    cfg.num_kv_heads = hkv;
    cfg.head_dim = D;
    PagedKVPool pool;
    REQUIRE(pool.initialize(cfg, 2, 170 * bs, bs, backend()).ok());
    BlockManager& mgr = pool.block_manager();
    const int slot = pool.acquire_slot();
    REQUIRE(slot >= 0);
    PagedKVCache& seq = pool.get_cache(slot);
    // a few blocks taken and given back first, so that the table is not the identity
    {
        PagedKVCache other(&mgr);
        REQUIRE(other.append_tokens(5 * bs));
        REQUIRE(seq.append_tokens(1));
        other.release();
        seq.truncate(0);
    }
    std::vector<std::vector<uint16_t>> want_k, want_v;
    for (int l = 0; l < layers; ++l) {
        want_k.push_back(download<uint16_t>(mgr.k_cache(l)));
        want_v.push_back(download<uint16_t>(mgr.v_cache(l)));
    }
    ChunkedPrefill driver;
    CHECK_CODE(driver.begin(10, 0), ErrorCode::InvalidState);
    REQUIRE(driver.initialize(&seq, 160, backend()).ok());
    driver.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
    CHECK_CODE(driver.begin(161 * bs, 512), ErrorCode::InvalidArgument);  // beyond the block table
    CHECK(seq.seq_len() == 0);

    struct Prompt {
        int tokens;
        uint32_t chunk_size;
        int expect_chunks;
    };
    uint32_t seed = 9100;
    int held = 0;
    for (const Prompt pr : {Prompt{2048, 512, 4}, Prompt{300, 128, 3}}) {
        REQUIRE(driver.begin(pr.tokens, pr.chunk_size).ok());
        CHECK(driver.num_chunks() == pr.expect_chunks);
        CHECK(driver.base_len() == held);
        CHECK(seq.seq_len() == held + pr.tokens);
        std::vector<int32_t> table(seq.block_table().begin(), seq.block_table().end());
        for (int l = 0; l < layers; ++l) {
            const int n = pr.tokens;
            auto q = randn(size_t(n) * hq * D, seed++), k = randn(size_t(n) * hkv * D, seed++),
                 v = randn(size_t(n) * hkv * D, seed++);
            Tensor Q = upload({n, hq, D}, DataType::FP32, q);
            Tensor K = upload({n, hkv, D}, DataType::FP32, k);
            Tensor V = upload({n, hkv, D}, DataType::FP32, v);
            Tensor O = Tensor::allocate({n, hq, D}, DataType::FP32, backend()).take();
            if (l == 0) {
                CHECK_OK(driver.run_layer(l, Q, K, V, O, scale, &rope));
            } else {  // chunk by chunk through run_chunk, on tensors of the chunk's own
                for (int c = 0; c < driver.num_chunks(); ++c) {
                    const int s0 = driver.chunk_start(c), len = driver.chunk_len(c);
                    auto part = [&](Tensor& t) { return t.slice(0, s0, s0 + len).take(); };
                    Tensor qc = part(Q), kc = part(K), vc = part(V), oc = part(O);
                    CHECK_OK(driver.run_chunk(l, c, qc, kc, vc, oc, scale, &rope));
                }
            }
            // oracle: the whole prompt at once
            CHECK(go_rope_apply(q.data(), n, hq, D, held, cos_t.data(), sin_t.data(), max_pos) == 0);
            CHECK(go_rope_apply(k.data(), n, hkv, D, held, cos_t.data(), sin_t.data(), max_pos) == 0);
            go_paged_kv_cache_append_f32(want_k[l].data(), transpose_heads(k, n).data(), table.data(), hkv, D,
                                         held, n, bs);
            go_paged_kv_cache_append_f32(want_v[l].data(), transpose_heads(v, n).data(), table.data(), hkv, D,
                                         held, n, bs);
            std::vector<float> want(q.size());
            go_attention_paged(q.data(), want_k[l].data(), want_v[l].data(), table.data(), bs, want.data(),
                               nullptr, 1, n, hq, hkv, D, held + n, held, scale);
            CHECK(download<float>(Q) == q);  // rotated at the right positions: the oracle's bits
            CHECK(download<float>(K) == k);
            CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);
            CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
            CHECK(close_enough(download<float>(O), want, "chunked prefill, paged"));
            for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
        }
        driver.finish();
        held += pr.tokens;
        CHECK(seq.seq_len() == held);
    }
    // the same 2048-token prompt again in chunks of 96 (22 chunks, the last of 32) into a
    // fresh sequence: identical pools row for row, outputs within tolerance of the oracle's
    {
        const int slot2 = pool.acquire_slot();
        REQUIRE(slot2 >= 0);
        PagedKVCache& seq2 = pool.get_cache(slot2);
        // not enough blocks left for 2048 tokens: begin() fails and gives everything back
        ChunkedPrefill d2;
        REQUIRE(d2.initialize(&seq2, 160, backend()).ok());
        const int free_before = pool.num_free_blocks();
        CHECK_CODE(d2.begin(2048, 96), ErrorCode::AllocationFailed);
        CHECK(seq2.seq_len() == 0 && pool.num_free_blocks() == free_before);
        seq.release();
        REQUIRE(d2.begin(2048, 96).ok());
        d2.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
        CHECK(d2.num_chunks() == 22 && d2.chunk_len(21) == 32 && d2.chunk_start(21) == 2016);
        std::vector<int32_t> table(seq2.block_table().begin(), seq2.block_table().end());
        const int n = 2048;
        auto q = randn(size_t(n) * hq * D, seed++), k = randn(size_t(n) * hkv * D, seed++),
             v = randn(size_t(n) * hkv * D, seed++);
        Tensor Q = upload({n, hq, D}, DataType::FP32, q);
        Tensor K = upload({n, hkv, D}, DataType::FP32, k);
        Tensor V = upload({n, hkv, D}, DataType::FP32, v);
        Tensor O = Tensor::allocate({n, hq, D}, DataType::FP32, backend()).take();
        CHECK_OK(d2.run_layer(0, Q, K, V, O, scale, &rope));
        CHECK(go_rope_apply(q.data(), n, hq, D, 0, cos_t.data(), sin_t.data(), max_pos) == 0);
        CHECK(go_rope_apply(k.data(), n, hkv, D, 0, cos_t.data(), sin_t.data(), max_pos) == 0);
        auto pk = download<uint16_t>(mgr.k_cache(0)), pv = download<uint16_t>(mgr.v_cache(0));
        auto wk = want_k[0], wv = want_v[0];
        go_paged_kv_cache_append_f32(wk.data(), transpose_heads(k, n).data(), table.data(), hkv, D, 0, n, bs);
        go_paged_kv_cache_append_f32(wv.data(), transpose_heads(v, n).data(), table.data(), hkv, D, 0, n, bs);
        CHECK(pk == wk);
        CHECK(pv == wv);
        std::vector<float> want(q.size());
        go_attention_paged(q.data(), wk.data(), wv.data(), table.data(), bs, want.data(), nullptr, 1, n, hq, hkv,
                           D, n, 0, scale);
        CHECK(close_enough(download<float>(O), want, "chunked prefill, 22 chunks of 96"));
        for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
    }

    // ---- contiguous KVCache, as the reference's loop runs it
    {
        const int max_seq = 700, n = 600;
        auto made = KVCache::allocate(cfg, max_seq, backend());
        REQUIRE(made.ok());
        KVCache cache = made.take();
        ChunkedPrefill d3;
        REQUIRE(d3.initialize(&cache, backend()).ok());
        d3.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
        CHECK_CODE(d3.begin(701, 256), ErrorCode::InvalidArgument);  // overflow (kv_cache.cpp:61-65)
        REQUIRE(d3.begin(n, 256).ok());
        CHECK(d3.num_chunks() == 3 && d3.chunk_len(2) == 88);
        for (int l = 0; l < layers; ++l) {
            auto q = randn(size_t(n) * hq * D, seed++), k = randn(size_t(n) * hkv * D, seed++),
                 v = randn(size_t(n) * hkv * D, seed++);
            Tensor Q = upload({n, hq, D}, DataType::FP32, q);
            Tensor K = upload({n, hkv, D}, DataType::FP32, k);
            Tensor V = upload({n, hkv, D}, DataType::FP32, v);
            Tensor O = Tensor::allocate({n, hq, D}, DataType::FP32, backend()).take();
            auto kv = cache.get(l);
            auto ck = download<uint16_t>(kv.first), cv = download<uint16_t>(kv.second);
            CHECK_OK(d3.run_layer(l, Q, K, V, O, scale, &rope));
            CHECK(cache.seq_len() == 0);  // advances after the last layer only
            CHECK(go_rope_apply(q.data(), n, hq, D, 0, cos_t.data(), sin_t.data(), max_pos) == 0);
            CHECK(go_rope_apply(k.data(), n, hkv, D, 0, cos_t.data(), sin_t.data(), max_pos) == 0);
            CHECK(go_kv_cache_append_f32(ck.data(), k.data(), hkv, D, 0, n, max_seq) == 0);
            CHECK(go_kv_cache_append_f32(cv.data(), v.data(), hkv, D, 0, n, max_seq) == 0);
            std::vector<float> want(q.size());
            go_attention_cached(q.data(), ck.data(), cv.data(), want.data(), nullptr, 1, n, hq, hkv, D, n, max_seq,
                                0, scale);
            CHECK(download<uint16_t>(kv.first) == ck);
            CHECK(download<uint16_t>(kv.second) == cv);
            CHECK(close_enough(download<float>(O), want, "chunked prefill, contiguous cache"));
            for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
        }
        d3.finish();
        CHECK(cache.seq_len() == n);
    }
}


// The projections either side of attention through HipCompute (MetalCompute::
// fused_qkv_matvec_q4k and matvec_q4k, include/granite/metal_compute.h:683-694, 73-79), one
// token and a batch of tokens, against the oracle's dequantise-and-multiply; and the scratch
// the batched form needs, reserved up front.
TEST_CASE(hip_compute_q4k_projections) {
    REQUIRE(backend() != nullptr);
    HipCompute* hc = get_hip_compute();
    REQUIRE(hc != nullptr);
    const int K = 1024, Nq = 256, Nkv = 64, batch = 40, blocks = K / 256;
    // random Q4_K super-blocks: any 144 bytes are a valid block once d and dmin are small halves
    std::mt19937 gen(4242);
    auto make_weights = [&](int rows) {
        std::vector<uint8_t> w(size_t(rows) * blocks * 144);
        for (auto& b : w) b = uint8_t(gen());
        for (size_t blk = 0; blk < w.size() / 144; ++blk) {
            const uint16_t d = go_fp32_to_fp16(3e-4f + 1e-6f * float(gen() % 400));
            const uint16_t dmin = go_fp32_to_fp16(2e-4f + 1e-6f * float(gen() % 400));
            std::memcpy(&w[blk * 144], &d, 2);
            std::memcpy(&w[blk * 144 + 2], &dmin, 2);
        }
        return w;
    };
    auto wq = make_weights(Nq), wk = make_weights(Nkv), wv = make_weights(Nkv);
    auto x = randn(size_t(batch) * K, 99);
    Tensor X = upload({batch, K}, DataType::FP32, x);
    Tensor WQ = upload({int64_t(wq.size())}, DataType::UINT8, wq);
    Tensor WK = upload({int64_t(wk.size())}, DataType::UINT8, wk);
    Tensor WV = upload({int64_t(wv.size())}, DataType::UINT8, wv);
    Tensor YQ = Tensor::allocate({batch, Nq}, DataType::FP32, backend()).take();
    Tensor YK = Tensor::allocate({batch, Nkv}, DataType::FP32, backend()).take();
    Tensor YV = Tensor::allocate({batch, Nkv}, DataType::FP32, backend()).take();
    auto ptr = [&](const Tensor& t) { return hip_device_pointer(backend(), t.buffer()); };

    auto check = [&](const Tensor& Y, const std::vector<uint8_t>& w, int N, int rows, const char* what) {
        std::vector<float> want(size_t(rows) * N);
        go_matvec_q4k(x.data(), w.data(), want.data(), K, N, rows);
        auto got = download<float>(Y);
        double worst = 0, scale = 0;
        for (size_t i = 0; i < want.size(); ++i) {
            worst = std::max(worst, std::fabs(double(got[i]) - double(want[i])));
            scale = std::max(scale, std::fabs(double(want[i])));
        }
        std::printf("  %s: max abs err %.3g (values up to %.3g)\n", what, worst, scale);
        CHECK(worst <= 1e-4 * std::max(scale, 1.0));  // float sums of K = 1024 products, two orders
    };
    // one token: the reference's signature
    CHECK_OK(hc->fused_qkv_matvec_q4k(ptr(X), ptr(WQ), ptr(WK), ptr(WV), ptr(YQ), ptr(YK), ptr(YV), K, Nq, Nkv));
    hc->sync();
    check(YQ, wq, Nq, 1, "fused qkv, one token (q)");
    check(YV, wv, Nkv, 1, "fused qkv, one token (v)");
    CHECK_OK(hc->matvec_q4k(ptr(X), ptr(WK), ptr(YK), K, Nkv));
    hc->sync();
    check(YK, wk, Nkv, 1, "matvec");
    // a batch of tokens, its scratch reserved first
    const size_t need = granite_hip_q4k_workspace_required(K, Nq + 2 * Nkv, batch);
    CHECK(need > 0);
    CHECK_OK(hc->reserve_workspace(need));
    const size_t held = hc->workspace_bytes();
    CHECK_OK(hc->fused_qkv_matvec_q4k_batched(ptr(X), ptr(WQ), ptr(WK), ptr(WV), ptr(YQ), ptr(YK), ptr(YV), K, Nq,
                                              Nkv, batch));
    hc->sync();
    CHECK(hc->workspace_bytes() == held);
    check(YQ, wq, Nq, batch, "fused qkv, 40 tokens (q)");
    check(YK, wk, Nkv, batch, "fused qkv, 40 tokens (k)");
    check(YV, wv, Nkv, batch, "fused qkv, 40 tokens (v)");
    CHECK_CODE(hc->matvec_q4k(ptr(X), ptr(WK), ptr(YK), 300, Nkv), ErrorCode::InvalidArgument);  // K % 256
    for (Tensor* t : {&X, &WQ, &WK, &WV, &YQ, &YK, &YV}) backend()->destroy_buffer(t->buffer());
}


TEST_CASE(speculative_commit_of_accepted_path) {
    REQUIRE(backend() != nullptr);
    PagedKVConfig cfg;
    cfg.block_size = 16;
    cfg.num_blocks = 10;
    cfg.num_layers = 2;
    cfg.num_kv_heads = 2;
    cfg.head_dim = D;
    BlockManager mgr;
    REQUIRE(mgr.initialize(cfg, backend()).ok());
    PagedKVCache seq(&mgr);
    const int original = 29, n_nodes = 7, hkv = 2, bs = 16;
    // as the runner does: the tree step reserved original + tree_size tokens
    REQUIRE(seq.append_tokens(original + n_nodes));
    SpeculationTree tree;
    tree.add_node(10, -1); tree.add_node(11, 0); tree.add_node(12, 0); tree.add_node(13, 1);
    tree.add_node(14, 1); tree.add_node(15, 2); tree.add_node(16, 4);
    const std::vector<int> accepted = tree.find_accepted_nodes({10, 11, 14, 16});
    REQUIRE((accepted == std::vector<int>{0, 1, 4, 6}));
    std::vector<Tensor> kt, vt;
    std::vector<std::vector<uint16_t>> kh, vh, want_k, want_v;
    for (int l = 0; l < 2; ++l) {
        kh.push_back(to_half(randn(size_t(hkv) * n_nodes * D, 8100 + l)));
        vh.push_back(to_half(randn(size_t(hkv) * n_nodes * D, 8200 + l)));
        kt.push_back(upload({hkv, n_nodes, D}, DataType::FP16, kh[l]));
        vt.push_back(upload({hkv, n_nodes, D}, DataType::FP16, vh[l]));
        want_k.push_back(download<uint16_t>(mgr.k_cache(l)));
        want_v.push_back(download<uint16_t>(mgr.v_cache(l)));
    }
    const int free_before = mgr.num_free_blocks();
    CHECK_OK(commit_tree_path(seq, original, accepted, kt, vt, backend()));
    CHECK(seq.seq_len() == original + 4);                       // 33 tokens: 3 blocks
    CHECK(seq.num_blocks() == 3 && mgr.num_free_blocks() >= free_before);
    for (int l = 0; l < 2; ++l) {
        for (int i = 0; i < 4; ++i) {
            const int pos = original + i;
            const size_t row = size_t(seq.block_table()[pos / bs]) * bs + pos % bs;
            for (int h = 0; h < hkv; ++h)
                for (int d = 0; d < D; ++d) {
                    want_k[l][(row * hkv + h) * D + d] = kh[l][(size_t(h) * n_nodes + accepted[i]) * D + d];
                    want_v[l][(row * hkv + h) * D + d] = vh[l][(size_t(h) * n_nodes + accepted[i]) * D + d];
                }
        }
        CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);   // bit exact, nothing else written
        CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
    }
    const int outside[1] = {n_nodes};
    CHECK_CODE(commit_tree_path(seq, original, outside, kt, vt, backend()), ErrorCode::InvalidArgument);
    // an empty path only restores the length
    CHECK_OK(commit_tree_path(seq, original, std::span<const int>(), kt, vt, backend()));
    CHECK(seq.seq_len() == original);
}

// Tree verification as SpeculativeRunner::verify_tree drives it (src/llm/speculative_runner.cpp:
// 586-674, 871-882) over a *paged* prefix: a prompt through ChunkedPrefill, a SpeculationTree
// built with add_node, tree attention for two layers (TransformerModel::attention_tree_gpu,
// src/llm/transformer.mm:2146-2402) against the oracle, the accepted path committed and the
// surplus blocks freed, and then one batched decode step whose output must be the oracle's
// on the committed sequence.
TEST_CASE(tree_verify_commit_then_decode_over_paged_prefix) {
    REQUIRE(backend() != nullptr);
    ModelConfig cfg;
    cfg.num_layers = 2;
    cfg.num_heads = 8;
    cfg.num_kv_heads = 2;
    cfg.head_dim = D;
    const int bs = 16, hq = 8, hkv = 2, max_blocks = 8, max_pos = max_blocks * bs, prompt = 45;
    PagedKVPool pool;
    REQUIRE(pool.initialize(cfg, 2, 12 * bs, bs, backend()).ok());
    BlockManager& mgr = pool.block_manager();
    RoPECache rope;
    rope.initialize(max_pos, D, 10000.0f);
    std::vector<float> cos_t(size_t(max_pos) * D / 2), sin_t(cos_t.size());
    go_rope_table(cos_t.data(), sin_t.data(), max_pos, D, 10000.0f);
    const float scale = 1.0f / std::sqrt(float(D));
    const int slot = pool.acquire_slot();
    REQUIRE(slot >= 0);
    PagedKVCache& seq = pool.get_cache(slot);
    uint32_t seed = 9100;

    // ---- the prefix: a prompt of 45 tokens in chunks of 32 (its parity is checked elsewhere)
    ChunkedPrefill prefill;
    REQUIRE(prefill.initialize(&seq, max_blocks, backend()).ok());
    prefill.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
    REQUIRE(prefill.begin(prompt, 32).ok());
    for (int l = 0; l < 2; ++l) {
        Tensor Q = upload({prompt, hq, D}, DataType::FP32, randn(size_t(prompt) * hq * D, seed++));
        Tensor K = upload({prompt, hkv, D}, DataType::FP32, randn(size_t(prompt) * hkv * D, seed++));
        Tensor V = upload({prompt, hkv, D}, DataType::FP32, randn(size_t(prompt) * hkv * D, seed++));
        Tensor O = Tensor::allocate({prompt, hq, D}, DataType::FP32, backend()).take();
        CHECK_OK(prefill.run_layer(l, Q, K, V, O, scale, &rope));
        (void)backend()->wait_for_completion();
        for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
    }
    prefill.finish();
    REQUIRE(seq.seq_len() == prompt);
    std::vector<std::vector<uint16_t>> want_k, want_v;  // the oracle's pools start from the device's bytes
    for (int l = 0; l < 2; ++l) {
        want_k.push_back(download<uint16_t>(mgr.k_cache(l)));
        want_v.push_back(download<uint16_t>(mgr.v_cache(l)));
    }

    // ---- the tree: 11 nodes, two branches under the root, depth 4
    SpeculationTree tree;
    tree.add_node(100, -1);                       // 0
    tree.add_node(101, 0); tree.add_node(102, 0); // 1 2
    tree.add_node(103, 1); tree.add_node(104, 1); // 3 4
    tree.add_node(105, 2);                        // 5
    tree.add_node(106, 4); tree.add_node(107, 4); // 6 7
    tree.add_node(108, 5);                        // 8
    tree.add_node(109, 7); tree.add_node(110, 3); // 9 10
    const std::vector<int> parents_int = tree.get_parent_indices();
    std::vector<int32_t> parents(parents_int.begin(), parents_int.end());
    const int N = int(tree.size());

    TreeVerify verify;
    CHECK_CODE(verify.begin(parents_int), ErrorCode::InvalidState);
    REQUIRE(verify.initialize(&seq, max_blocks, 16, backend()).ok());
    const int bad_parent[2] = {-1, 5};
    CHECK_CODE(verify.begin(bad_parent), ErrorCode::InvalidArgument);
    REQUIRE(verify.begin(parents_int).ok());
    CHECK(verify.original_len() == prompt && verify.num_nodes() == N);
    CHECK(seq.seq_len() == prompt);  // nothing is appended by the tree step
    const int accepted_before_layers[1] = {0};
    CHECK_CODE(verify.commit(accepted_before_layers), ErrorCode::InvalidState);

    std::vector<int32_t> table(seq.block_table().begin(), seq.block_table().end());
    std::vector<std::vector<uint16_t>> node_k, node_v;  // per layer [N, Hkv, D] halves (truncated)
    for (int l = 0; l < 2; ++l) {
        auto q = randn(size_t(N) * hq * D, seed++), k = randn(size_t(N) * hkv * D, seed++),
             v = randn(size_t(N) * hkv * D, seed++);
        Tensor Q = upload({N, hq, D}, DataType::FP32, q);
        Tensor K = upload({N, hkv, D}, DataType::FP32, k);
        Tensor V = upload({N, hkv, D}, DataType::FP32, v);
        Tensor O = Tensor::allocate({N, hq, D}, DataType::FP32, backend()).take();
        CHECK_OK(verify.run_layer(l, Q, K, V, O, scale));
        // oracle: the tree's K/V as the cast leaves them (transformer.mm:2295-2304), floats [N, Hkv, D]
        node_k.push_back(to_half(k));
        node_v.push_back(to_half(v));
        auto kf = to_float(node_k[l]), vf = to_float(node_v[l]);
        std::vector<float> want(q.size());
        CHECK(go_attention_tree(q.data(), want_k[l].data(), want_v[l].data(), table.data(), bs, 0, kf.data(),
                                vf.data(), parents.data(), want.data(), nullptr, 1, N, hq, hkv, D, prompt,
                                scale) == 0);
        CHECK(close_enough(download<float>(O), want, "tree attention over the paged prefix"));
        // the kept copy is [Hkv, N, D], bit for bit the truncated rows
        auto kept = download<uint16_t>(verify.k_tree(l));
        bool same = kept.size() == node_k[l].size();
        for (int h = 0; h < hkv && same; ++h)
            for (int n = 0; n < N && same; ++n)
                for (int d = 0; d < D; ++d)
                    same = same && kept[(size_t(h) * N + n) * D + d] == node_k[l][(size_t(n) * hkv + h) * D + d];
        CHECK(same);
        for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
    }

    // ---- the target agrees with 100, 101, 104, 107 and then says 555 where the tree says 109
    const std::vector<int32_t> target_choices = {100, 101, 104, 107, 555};
    const std::vector<int> accepted = tree.find_accepted_nodes(target_choices);
    REQUIRE((accepted == std::vector<int>{0, 1, 4, 7}));
    const int free_before = mgr.num_free_blocks();
    CHECK_OK(verify.commit(accepted));
    const int committed = prompt + int(accepted.size());  // 49 tokens: 4 blocks
    CHECK(seq.seq_len() == committed && seq.num_blocks() == 4);
    CHECK(mgr.num_free_blocks() == free_before - 1);      // 45 tokens held 3 blocks
    table.assign(seq.block_table().begin(), seq.block_table().end());
    for (int l = 0; l < 2; ++l) {
        for (size_t i = 0; i < accepted.size(); ++i) {
            const int pos = prompt + int(i);
            const size_t row = size_t(table[pos / bs]) * bs + pos % bs;
            for (int h = 0; h < hkv; ++h)
                for (int d = 0; d < D; ++d) {
                    want_k[l][(row * hkv + h) * D + d] = node_k[l][(size_t(accepted[i]) * hkv + h) * D + d];
                    want_v[l][(row * hkv + h) * D + d] = node_v[l][(size_t(accepted[i]) * hkv + h) * D + d];
                }
        }
        CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);  // bit exact, nothing else written
        CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
    }
    CHECK_CODE(verify.commit(accepted), ErrorCode::InvalidState);  // one commit per begin()

    // ---- the next decode step sees prompt + accepted path
    PagedDecodeBatch step;
    REQUIRE(step.initialize(&pool, 2, max_blocks, backend()).ok());
    step.set_rounding(GRANITE_HIP_ROUND_TRUNCATE);
    const int slots[1] = {slot};
    auto failed = step.begin_step(slots);
    REQUIRE(failed.ok() && failed.value().empty());
    CHECK(seq.seq_len() == committed + 1);
    std::vector<int32_t> tables(max_blocks, 0), seq_lens = {committed + 1};
    std::copy(seq.block_table().begin(), seq.block_table().end(), tables.begin());
    for (int l = 0; l < 2; ++l) {
        auto q = randn(size_t(hq) * D, seed++), k = randn(size_t(hkv) * D, seed++), v = randn(size_t(hkv) * D, seed++);
        Tensor Q = upload({1, hq, D}, DataType::FP32, q);
        Tensor K = upload({1, hkv, D}, DataType::FP32, k);
        Tensor V = upload({1, hkv, D}, DataType::FP32, v);
        Tensor O = Tensor::allocate({1, hq, D}, DataType::FP32, backend()).take();
        CHECK_OK(step.run_layer(l, Q, K, V, O, scale, &rope));
        CHECK(go_rope_apply(q.data(), 1, hq, D, committed, cos_t.data(), sin_t.data(), max_pos) == 0);
        CHECK(go_rope_apply(k.data(), 1, hkv, D, committed, cos_t.data(), sin_t.data(), max_pos) == 0);
        go_paged_kv_cache_append_f32(want_k[l].data(), k.data(), tables.data(), hkv, D, committed, 1, bs);
        go_paged_kv_cache_append_f32(want_v[l].data(), v.data(), tables.data(), hkv, D, committed, 1, bs);
        std::vector<float> want(q.size());
        go_batched_paged_decode(q.data(), want_k[l].data(), want_v[l].data(), tables.data(), seq_lens.data(),
                                want.data(), nullptr, 1, hq, hkv, D, bs, max_blocks, scale);
        CHECK(download<uint16_t>(mgr.k_cache(l)) == want_k[l]);
        CHECK(download<uint16_t>(mgr.v_cache(l)) == want_v[l]);
        CHECK(close_enough(download<float>(O), want, "decode step after the commit"));
        for (Tensor* t : {&Q, &K, &V, &O}) backend()->destroy_buffer(t->buffer());
    }
}

// A chunk that fails (wrong tensor shape) leaves a paged prompt open with its tokens already
// taken; abort() gives them back, and a new begin() does the same by itself.
TEST_CASE(chunked_prefill_abort_after_failed_chunk) {
    REQUIRE(backend() != nullptr);
    PagedKVConfig cfg;
    cfg.block_size = 16;
    cfg.num_blocks = 8;
    cfg.num_layers = 1;
    cfg.num_kv_heads = 2;
    cfg.head_dim = D;
    BlockManager mgr;
    REQUIRE(mgr.initialize(cfg, backend()).ok());
    PagedKVCache seq(&mgr);
    REQUIRE(seq.append_tokens(20));  // an earlier prefix: 2 blocks
    const int free_before = mgr.num_free_blocks();
    ChunkedPrefill prefill;
    REQUIRE(prefill.initialize(&seq, 8, backend()).ok());
    REQUIRE(prefill.begin(70, 32).ok());
    CHECK(prefill.is_open() && prefill.base_len() == 20 && seq.seq_len() == 90);
    Tensor wrong = Tensor::allocate({5, 4, D}, DataType::FP32, backend()).take();  // the chunk has 32 rows
    CHECK_CODE(prefill.run_chunk(0, 0, wrong, wrong, wrong, wrong, 0.1f, nullptr), ErrorCode::ShapeMismatch);
    CHECK(prefill.is_open() && seq.seq_len() == 90);  // still covers rows nobody wrote
    prefill.abort();
    CHECK(!prefill.is_open() && seq.seq_len() == 20 && seq.num_blocks() == 2);
    CHECK(mgr.num_free_blocks() == free_before);
    prefill.abort();  // nothing open: no effect
    CHECK(seq.seq_len() == 20);
    // a new begin() on a prompt left open aborts it first
    REQUIRE(prefill.begin(40, 0).ok());
    CHECK(seq.seq_len() == 60);
    REQUIRE(prefill.begin(10, 0).ok());
    CHECK(prefill.base_len() == 20 && seq.seq_len() == 30);
    prefill.finish();
    CHECK(!prefill.is_open() && seq.seq_len() == 30);
    backend()->destroy_buffer(wrong.buffer());
}

int main(int argc, char** argv) {
    if (!backend()) {
        std::printf("no usable gfx950 GPU: skipping\n");
        return 77;
    }
    return hosttest::run_all(argc, argv);
}
