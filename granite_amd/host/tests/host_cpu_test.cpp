// Host-side logic that needs no GPU: Result/Error plumbing, Tensor, the
// operator registry, KV bookkeeping (KVCache checks, BlockManager, PagedKVCache,
// pools) and SpeculationTree.  The KVCache cases repeat the reference's own
// (tests/test_llm.cpp:113-160) on a host-memory test double.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "check.h"
#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite/kv_cache.h"
#include "granite/operators.h"
#include "granite/paged_batch.h"
#include "granite/rope.h"
#include "granite/tree_verify.h"
#include "granite_hip.h"
#include "host_memory_backend.h"

extern "C" {
// CPU oracle's restatement of the block bookkeeping (oracle/granite_oracle.c),
// linked as the checker of paged_bookkeeping_matches_oracle.
struct go_block_manager;
struct go_paged_cache;
go_block_manager* go_block_manager_new(int num_blocks, int block_size);
void go_block_manager_delete(go_block_manager* m);
int go_block_manager_num_free(const go_block_manager* m);
go_paged_cache* go_paged_cache_new(go_block_manager* mgr);
void go_paged_cache_delete(go_paged_cache* c);
int go_paged_cache_append_tokens(go_paged_cache* c, int num_tokens);
void go_paged_cache_truncate(go_paged_cache* c, int new_len);
void go_paged_cache_release(go_paged_cache* c);
int go_paged_cache_seq_len(const go_paged_cache* c);
int go_paged_cache_num_blocks(const go_paged_cache* c);
const int* go_paged_cache_table(const go_paged_cache* c);
int go_paged_cache_physical_block(const go_paged_cache* c, int pos);
}

using namespace granite;
using hosttest::HostMemoryBackend;

static Result<int> half_of(int v) {
    if (v % 2) return Error(ErrorCode::InvalidArgument, "odd");
    return v / 2;
}
static Result<int> quarter_of(int v) {
    GRANITE_TRY_ASSIGN(h, half_of(v));
    GRANITE_TRY_ASSIGN(q, half_of(h));
    return q;
}

TEST_CASE(result_and_error) {
    CHECK(quarter_of(8).ok() && quarter_of(8).value() == 2);
    CHECK_CODE(quarter_of(6), ErrorCode::InvalidArgument);
    Result<void> fine;
    CHECK(fine.ok());
    Result<void> bad(ErrorCode::Timeout);
    CHECK(!bad.ok() && bad.error().code() == ErrorCode::Timeout);
    CHECK(std::string(error_code_name(ErrorCode::NotImplemented)) == "NotImplemented");
    CHECK(static_cast<int>(ErrorCode::NotImplemented) == 25);
    CHECK(half_of(3).value_or(-1) == -1);
    CHECK(half_of(4).map([](int v) { return v + 1; }).value() == 3);
    CHECK(Error(ErrorCode::InvalidShape, "x").to_string().find("InvalidShape: x") == 0);
}

TEST_CASE(enum_values_match_reference_order) {
    CHECK(static_cast<int>(DataType::FP16) == 1);
    CHECK(static_cast<int>(DataType::UINT4) == 10);
    CHECK(static_cast<int>(BackendType::Talos) == 3);
    CHECK(static_cast<int>(BackendType::HIP) == 4);
    CHECK(static_cast<int>(MemoryType::Managed) == 2);
    CHECK(static_cast<int>(OpType::ScaledDotProductAttention) == 35);
    CHECK(static_cast<int>(OpType::Custom) == 42);
    CHECK(std::string(op_type_name(OpType::ScaledDotProductAttention)) ==
          "ScaledDotProductAttention");
    CHECK(std::string(op_type_name(OpType::Custom)) == "Custom");
    CHECK(std::string(backend_name(BackendType::HIP)) == "HIP");
    CHECK(dtype_size(DataType::FP16) == 2 && dtype_size(DataType::INT64) == 8);
    CHECK(GRANITE_HIP_MEM_MANAGED == static_cast<int>(MemoryType::Managed));
}

TEST_CASE(status_codes_map_to_error_codes) {
    CHECK(hip_status_to_result(GRANITE_HIP_OK, "x").ok());
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_EINVAL, "x"), ErrorCode::InvalidArgument);
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_ENOTINIT, "x"), ErrorCode::BackendNotInitialized);
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_ENOMEM, "x"), ErrorCode::AllocationFailed);
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_EUNSUPPORTED, "x"), ErrorCode::NotImplemented);
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_ENULL, "x"), ErrorCode::NullPointer);
    CHECK_CODE(hip_status_to_result(GRANITE_HIP_EOVERFLOW, "x"), ErrorCode::InvalidArgument);
    CHECK_CODE(hip_status_to_result(719, "x"), ErrorCode::ExecutionFailed);
}

TEST_CASE(tensor_allocate_errors) {
    HostMemoryBackend be;
    const int64_t shape[2] = {4, 8};
    CHECK_CODE(Tensor::allocate(shape, DataType::FP32, nullptr), ErrorCode::NullPointer);
    CHECK_CODE(Tensor::allocate(shape, DataType::FP32, &be), ErrorCode::BackendNotInitialized);
    CHECK_OK(be.initialize());
    CHECK_CODE(Tensor::allocate(std::span<const int64_t>{}, DataType::FP32, &be),
               ErrorCode::InvalidShape);
    const int64_t zero[2] = {4, 0};
    CHECK_CODE(Tensor::allocate(zero, DataType::FP32, &be), ErrorCode::InvalidShape);
    const int64_t neg[2] = {-1, 3};
    CHECK_CODE(Tensor::allocate(neg, DataType::FP32, &be), ErrorCode::InvalidShape);
    be.max_buffer = 100;
    CHECK_CODE(Tensor::allocate(shape, DataType::FP32, &be), ErrorCode::OutOfMemory);
    be.max_buffer = 128;
    CHECK_OK(Tensor::allocate(shape, DataType::FP32, &be));
}

TEST_CASE(tensor_views_and_slices) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    auto made = Tensor::allocate({2, 3, 4}, DataType::FP16, &be);
    REQUIRE(made.ok());
    Tensor t = made.take();
    CHECK(t.ndim() == 3 && t.numel() == 24 && t.size_bytes() == 48);
    CHECK(t.size(-1) == 4 && t.size(-2) == 3 && t.size(0) == 2);
    CHECK(t.strides()[0] == 12 && t.strides()[1] == 4 && t.strides()[2] == 1);
    CHECK(t.is_contiguous() && t.valid());
    auto p = t.data<uint16_t>();
    REQUIRE(p.ok());
    for (int i = 0; i < 24; ++i) p.value()[i] = static_cast<uint16_t>(i);
    t.unmap();

    const int64_t flat[2] = {6, 4};
    auto v = t.view(flat);
    REQUIRE(v.ok());
    CHECK(v.value().buffer() == t.buffer() && v.value().size(0) == 6);
    const int64_t wrong[2] = {5, 4};
    CHECK_CODE(t.view(wrong), ErrorCode::ShapeMismatch);

    auto s = t.slice(0, 1, 2);
    REQUIRE(s.ok());
    CHECK(s.value().buffer_offset() == 24 && s.value().size(0) == 1);
    CHECK(s.value().data<uint16_t>().value()[0] == 12);
    auto mid = t.slice(1, 1, 3);
    REQUIRE(mid.ok());
    CHECK(!mid.value().is_contiguous());
    CHECK_CODE(mid.value().view(flat), ErrorCode::InvalidState);
    CHECK_CODE(t.slice(3, 0, 1), ErrorCode::InvalidArgument);
    CHECK_CODE(t.slice(0, 1, 3), ErrorCode::InvalidArgument);

    auto c = t.clone();
    REQUIRE(c.ok());
    CHECK(c.value().buffer() != t.buffer());
    CHECK(std::memcmp(c.value().data<uint16_t>().value(), p.value(), 48) == 0);
    auto other = Tensor::allocate({2, 3, 4}, DataType::FP32, &be).take();
    CHECK_CODE(other.copy_from(t), ErrorCode::DTypeMismatch);
    Tensor none;
    CHECK(!none.valid() && none.empty());
    CHECK_CODE(none.data<float>(), ErrorCode::InvalidState);
}

namespace {
struct FakeOp final : IOperator {
    int tag;
    explicit FakeOp(int t) : tag(t) {}
    OpType type() const override { return OpType::Softmax; }
    Result<void> validate(const OpContext&) const override { return {}; }
    Result<std::vector<std::vector<int64_t>>> infer_shapes(const OpContext&) const override {
        return std::vector<std::vector<int64_t>>{{tag}};
    }
    Result<void> execute(OpContext&) override { return {}; }
};
int tag_of(IOperator* op) {
    OpContext ctx;
    return static_cast<int>(op->infer_shapes(ctx).value()[0][0]);
}
}  // namespace

TEST_CASE(operator_registry) {
    auto& reg = OperatorRegistry::instance();
    CHECK(reg.create(OpType::Softmax, BackendType::HIP) == nullptr);
    reg.register_op(OpType::Softmax, BackendType::CPU, [] { return std::make_unique<FakeOp>(1); });
    auto via_fallback = reg.create(OpType::Softmax, BackendType::HIP);  // CPU factory
    REQUIRE(via_fallback != nullptr);
    CHECK(tag_of(via_fallback.get()) == 1);
    CHECK(!reg.has_implementation(OpType::Softmax, BackendType::HIP));
    reg.register_op(OpType::Softmax, BackendType::HIP, [] { return std::make_unique<FakeOp>(2); });
    CHECK(tag_of(reg.create(OpType::Softmax, BackendType::HIP).get()) == 2);
    reg.register_op(OpType::Softmax, BackendType::HIP, [] { return std::make_unique<FakeOp>(3); });
    CHECK(tag_of(reg.create(OpType::Softmax, BackendType::HIP).get()) == 3);  // replaced
    CHECK(reg.create(OpType::MatMul, BackendType::HIP) == nullptr);

    register_hip_operators();
    register_hip_operators();  // idempotent
    CHECK(reg.has_implementation(OpType::ScaledDotProductAttention, BackendType::HIP));
    auto ops = reg.get_ops_for_backend(BackendType::HIP);
    CHECK(std::count(ops.begin(), ops.end(), OpType::ScaledDotProductAttention) == 1);
    auto attn = reg.create(OpType::ScaledDotProductAttention, BackendType::HIP);
    REQUIRE(attn != nullptr);
    CHECK(attn->type() == OpType::ScaledDotProductAttention);
    CHECK(!attn->can_fuse_with(OpType::Add));
}

TEST_CASE(attention_op_validation) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    register_hip_operators();
    auto op = OperatorRegistry::instance().create(OpType::ScaledDotProductAttention,
                                                  BackendType::HIP);
    REQUIRE(op != nullptr);
    OpContext ctx;
    ctx.backend = &be;
    auto q = Tensor::allocate({8, 4, 128}, DataType::FP16, &be).take();
    auto k = Tensor::allocate({2, 9, 128}, DataType::FP16, &be).take();
    auto v = Tensor::allocate({2, 9, 128}, DataType::FP16, &be).take();
    ctx.inputs = {q, k};
    CHECK_CODE(op->validate(ctx), ErrorCode::InvalidArgument);  // needs Q, K, V
    ctx.inputs = {q, k, v};
    CHECK_OK(op->validate(ctx));
    auto shapes = op->infer_shapes(ctx);
    REQUIRE(shapes.ok());
    CHECK((shapes.value() == std::vector<std::vector<int64_t>>{{8, 4, 128}}));

    auto k32 = Tensor::allocate({2, 9, 128}, DataType::FP32, &be).take();
    ctx.inputs = {q, k32, v};
    CHECK_CODE(op->validate(ctx), ErrorCode::DTypeMismatch);  // K and V of different types
    auto v32 = Tensor::allocate({2, 9, 128}, DataType::FP32, &be).take();
    ctx.inputs = {q, k32, v32};
    CHECK_OK(op->validate(ctx));  // both float: rounded to half on the way in
    auto k3 = Tensor::allocate({3, 9, 128}, DataType::FP16, &be).take();
    auto v3 = Tensor::allocate({3, 9, 128}, DataType::FP16, &be).take();
    ctx.inputs = {q, k3, v3};
    CHECK_CODE(op->validate(ctx), ErrorCode::ShapeMismatch);  // 8 % 3 != 0
    auto vshort = Tensor::allocate({2, 8, 128}, DataType::FP16, &be).take();
    ctx.inputs = {q, k, vshort};
    CHECK_CODE(op->validate(ctx), ErrorCode::ShapeMismatch);

    // On a non-HIP backend the operator refuses to run: there is no host path.
    ctx.inputs = {q, k, v};
    ctx.outputs = {Tensor::allocate({8, 4, 128}, DataType::FP16, &be).take()};
    CHECK_CODE(op->execute(ctx), ErrorCode::BackendNotSupported);
}

TEST_CASE(kv_cache_allocation_and_checks) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    ModelConfig cfg;
    cfg.num_layers = 2;
    cfg.num_kv_heads = 4;
    cfg.head_dim = 64;
    cfg.num_heads = 8;
    auto made = KVCache::allocate(cfg, 512, &be);
    REQUIRE(made.ok());
    KVCache cache = made.take();
    CHECK(cache.is_allocated());
    CHECK(cache.max_seq_len() == 512 && cache.seq_len() == 0);
    CHECK(cache.memory_bytes() == size_t(2) * 2 * 4 * 512 * 64 * 2);
    auto [k0, v0] = cache.get(0);
    CHECK(k0.valid() && v0.valid() && k0.ndim() == 4 && k0.size(2) == 512 && k0.size(0) == 1);
    auto [kx, vx] = cache.get(2);
    CHECK(!kx.valid() && !vx.valid());

    auto nk = Tensor::allocate({1, 4, 3, 64}, DataType::FP16, &be).take();
    auto nv = Tensor::allocate({1, 4, 3, 64}, DataType::FP16, &be).take();
    CHECK_CODE(cache.append(-1, nk, nv), ErrorCode::InvalidArgument);
    CHECK_CODE(cache.append(2, nk, nv), ErrorCode::InvalidArgument);
    cache.set_seq_len(510);
    CHECK_CODE(cache.append(0, nk, nv), ErrorCode::InvalidArgument);  // 510 + 3 > 512
    CHECK(cache.append(0, nk, nv).error().message().find("KV cache overflow: 510 + 3 > 512") == 0);
    cache.set_seq_len(0);
    // The bytes move on the GPU only; a non-HIP backend is refused, not emulated.
    CHECK_CODE(cache.append(0, nk, nv), ErrorCode::BackendNotSupported);
    auto bad = Tensor::allocate({1, 2, 3, 64}, DataType::FP16, &be).take();
    CHECK_CODE(cache.append(0, bad, bad), ErrorCode::ShapeMismatch);

    cache.increment_seq_len(7);
    CHECK(cache.seq_len() == 7);
    cache.truncate(9);
    CHECK(cache.seq_len() == 7);
    cache.truncate(-1);
    CHECK(cache.seq_len() == 7);
    cache.truncate(4);
    CHECK(cache.seq_len() == 4);
    cache.clear();
    CHECK(cache.seq_len() == 0);

    KVCache empty;
    CHECK(!empty.is_allocated() && empty.memory_bytes() == 0);
    be.shutdown();
    CHECK_CODE(KVCache::allocate(cfg, 8, &be), ErrorCode::BackendNotInitialized);
}

TEST_CASE(kv_cache_pool_slots) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    ModelConfig cfg;
    cfg.num_layers = 1;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 32;
    KVCachePool pool;
    CHECK_OK(pool.allocate(3, cfg, 16, &be));
    CHECK(pool.num_slots() == 3 && pool.num_free_slots() == 3);
    CHECK(pool.acquire_slot() == 0 && pool.acquire_slot() == 1);
    pool.get_cache(1).set_seq_len(5);
    pool.release_slot(1);
    CHECK(!pool.is_slot_in_use(1) && pool.is_slot_in_use(0));
    CHECK(pool.acquire_slot() == 1);
    CHECK(pool.get_cache(1).seq_len() == 0);  // cleared on acquire
    CHECK(pool.acquire_slot() == 2 && pool.acquire_slot() == -1);
    pool.release_slot(7);
    pool.release_slot(-1);
    CHECK(pool.num_free_slots() == 0);
}

TEST_CASE(block_manager_is_lifo) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    BlockManager mgr;
    PagedKVConfig cfg;
    cfg.num_blocks = 0;
    CHECK_CODE(mgr.initialize(cfg, &be), ErrorCode::InvalidArgument);
    cfg.num_blocks = 4;
    cfg.block_size = 0;
    CHECK_CODE(mgr.initialize(cfg, &be), ErrorCode::InvalidArgument);
    cfg.block_size = 16;
    cfg.num_layers = 2;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 8;
    CHECK(!mgr.is_initialized());
    CHECK_OK(mgr.initialize(cfg, &be));
    CHECK(mgr.is_initialized() && mgr.num_total_blocks() == 4 && mgr.block_size() == 16);
    CHECK(mgr.k_cache(1).size(0) == 64 && mgr.k_cache(1).size(1) == 2 && mgr.v_cache(0).size(2) == 8);
    CHECK(mgr.k_cache(0).dtype() == DataType::FP16);
    // the stack hands out the highest index first
    CHECK(mgr.allocate_block() == 3 && mgr.allocate_block() == 2);
    CHECK(mgr.num_free_blocks() == 2);
    mgr.free_block(3);
    mgr.free_block(3);   // double free ignored
    mgr.free_block(9);   // out of range ignored
    mgr.free_block(-1);
    mgr.free_block(0);   // never handed out: ignored
    CHECK(mgr.num_free_blocks() == 3);
    CHECK(mgr.allocate_block() == 3);  // freed last, reused first
    CHECK(mgr.allocate_block() == 1 && mgr.allocate_block() == 0);
    CHECK(mgr.allocate_block() == -1 && mgr.num_free_blocks() == 0);
    cfg.num_layers = 1;
    be.max_buffer = 16;
    BlockManager starved;
    CHECK_CODE(starved.initialize(cfg, &be), ErrorCode::AllocationFailed);
}

TEST_CASE(paged_cache_block_tables) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    BlockManager mgr;
    PagedKVConfig cfg{16, 6, 1, 1, 8};
    CHECK_OK(mgr.initialize(cfg, &be));
    PagedKVCache a(&mgr), b(&mgr), detached;
    CHECK(!detached.append_tokens(1) && detached.get_physical_block(0) == -1 &&
          detached.get_block_offset(5) == 0);
    CHECK(a.append_tokens(1));
    CHECK(a.seq_len() == 1 && a.num_blocks() == 1 && a.block_table()[0] == 5);
    CHECK(a.append_tokens(15) && a.num_blocks() == 1);  // exactly one full block
    CHECK(a.append_tokens(1) && a.num_blocks() == 2 && a.block_table()[1] == 4);
    CHECK(b.append_tokens(40) && b.num_blocks() == 3);
    CHECK((b.block_table() == std::vector<int>{3, 2, 1}));
    CHECK(a.get_physical_block(16) == 4 && a.get_block_offset(16) == 0);
    CHECK(a.get_physical_block(15) == 5 && a.get_block_offset(15) == 15);
    CHECK(a.get_physical_block(32) == -1);
    // pool has one block left: a request for three more takes it and fails,
    // keeping the length (src/llm/paged_kv_cache.cpp:120-145)
    CHECK(!a.append_tokens(48));
    CHECK(a.seq_len() == 17 && a.num_blocks() == 3 && mgr.num_free_blocks() == 0);
    a.truncate(20);  // not shorter: nothing happens
    CHECK(a.seq_len() == 17 && a.num_blocks() == 3);
    a.truncate(16);
    CHECK(a.seq_len() == 16 && a.num_blocks() == 1 && mgr.num_free_blocks() == 2);
    a.truncate(0);
    CHECK(a.seq_len() == 0 && a.num_blocks() == 0 && mgr.num_free_blocks() == 3);
    b.clear();
    CHECK(b.seq_len() == 0 && mgr.num_free_blocks() == 6);
    // blocks come back in the order they were freed
    CHECK(a.append_tokens(1) && a.block_table()[0] == 1);
}

// A long random trace of grow / truncate / release over five sequences sharing
// a small pool: every block table and the free count must agree with the
// oracle's restatement after every step.
TEST_CASE(paged_bookkeeping_matches_oracle) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    const int num_blocks = 37, bs = 8, nseq = 5;
    BlockManager mgr;
    PagedKVConfig cfg{bs, num_blocks, 1, 1, 8};
    CHECK_OK(mgr.initialize(cfg, &be));
    go_block_manager* omgr = go_block_manager_new(num_blocks, bs);
    std::vector<PagedKVCache> seqs(nseq, PagedKVCache(&mgr));
    std::vector<go_paged_cache*> oseqs;
    for (int i = 0; i < nseq; ++i) oseqs.push_back(go_paged_cache_new(omgr));
    uint64_t state = 0x9e3779b97f4a7c15ull;
    auto next = [&](uint32_t mod) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return uint32_t(state >> 33) % mod;
    };
    int mismatches = 0, refusals = 0;
    for (int step = 0; step < 4000; ++step) {
        const int i = int(next(nseq));
        const uint32_t what = next(10);
        if (what < 6) {
            const int n = int(next(40));
            const bool ok = seqs[i].append_tokens(n);
            const int want = go_paged_cache_append_tokens(oseqs[i], n);
            mismatches += ok != (want != 0);
            refusals += !ok;
        } else if (what < 9) {
            const int to = int(next(uint32_t(seqs[i].seq_len() + 5)));
            seqs[i].truncate(to);
            go_paged_cache_truncate(oseqs[i], to);
        } else {
            seqs[i].release();
            go_paged_cache_release(oseqs[i]);
        }
        mismatches += mgr.num_free_blocks() != go_block_manager_num_free(omgr);
        for (int s = 0; s < nseq; ++s) {
            mismatches += seqs[s].seq_len() != go_paged_cache_seq_len(oseqs[s]);
            mismatches += seqs[s].num_blocks() != go_paged_cache_num_blocks(oseqs[s]);
            if (seqs[s].num_blocks() == go_paged_cache_num_blocks(oseqs[s]) && seqs[s].num_blocks())
                mismatches += std::memcmp(seqs[s].block_table().data(), go_paged_cache_table(oseqs[s]),
                                          sizeof(int) * size_t(seqs[s].num_blocks())) != 0;
            const int probe = int(next(400));
            mismatches += seqs[s].get_physical_block(probe) !=
                          go_paged_cache_physical_block(oseqs[s], probe);
        }
    }
    CHECK(mismatches == 0);
    CHECK(refusals > 0);  // the trace did exhaust the pool
    for (auto* c : oseqs) go_paged_cache_delete(c);
    go_block_manager_delete(omgr);
}

TEST_CASE(paged_pool_slots) {
    HostMemoryBackend be;
    CHECK_OK(be.initialize());
    ModelConfig cfg;
    cfg.num_layers = 2;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 16;
    PagedKVPool pool;
    CHECK(!pool.is_initialized());
    CHECK_OK(pool.initialize(cfg, /*max_sequences*/ 2, /*max_total_tokens*/ 100, /*block*/ 16, &be));
    CHECK(pool.is_initialized() && pool.num_free_blocks() == 7 && pool.num_free_slots() == 2);
    int s0 = pool.acquire_slot(), s1 = pool.acquire_slot();
    CHECK(s0 == 0 && s1 == 1 && pool.acquire_slot() == -1);
    CHECK(pool.get_cache(s0).block_manager() == &pool.block_manager());
    CHECK(pool.get_cache(s0).append_tokens(33));
    CHECK(pool.num_free_blocks() == 4);
    pool.release_slot(s0);
    CHECK(pool.num_free_blocks() == 7 && pool.num_free_slots() == 1);
    pool.release_slot(s0);  // already free: nothing happens
    pool.release_slot(5);
    CHECK(pool.acquire_slot() == 0 && pool.get_cache(0).seq_len() == 0);
}

TEST_CASE(speculation_tree) {
    SpeculationTree tree;
    CHECK(tree.size() == 0 && tree.flatten_tokens().empty());
    CHECK(tree.find_accepted_path({1, 2}).empty());
    //        0:10
    //       /    \        .
    //    1:11    2:12
    //    /  \       \     .
    //  3:13 4:14    5:15
    //          \          .
    //          6:16
    CHECK(tree.add_node(10, -1) == 0);
    CHECK(tree.add_node(11, 0, -0.5f) == 1);
    CHECK(tree.add_node(12, 0) == 2);
    CHECK(tree.add_node(13, 1) == 3);
    CHECK(tree.add_node(14, 1) == 4);
    CHECK(tree.add_node(15, 2) == 5);
    CHECK(tree.add_node(16, 4) == 6);
    CHECK(tree.size() == 7 && tree.max_depth() == 3);
    CHECK(tree.node(6).depth == 3 && tree.node(1).log_prob == -0.5f);
    CHECK(tree.get_node(7) == nullptr && tree.get_node(-1) == nullptr &&
          tree.get_node(2)->token == 12);
    CHECK((tree.get_parent_indices() == std::vector<int>{-1, 0, 0, 1, 1, 2, 4}));
    CHECK((tree.get_leaves() == std::vector<int>{3, 5, 6}));
    CHECK((tree.get_path(6) == std::vector<int>{0, 1, 4, 6}));
    CHECK((tree.get_path(0) == std::vector<int>{0}));
    CHECK((tree.flatten_tokens() == std::vector<int32_t>{10, 11, 12, 13, 14, 15, 16}));

    using P = std::vector<int32_t>;
    CHECK((tree.find_accepted_path({10, 11, 14, 16}) == P{10, 11, 14, 16}));
    CHECK((tree.find_accepted_path({10, 12, 15, 99}) == P{10, 12, 15}));   // leaf reached
    CHECK((tree.find_accepted_path({10, 11, 99, 5}) == P{10, 11, 99}));    // target's token closes
    CHECK((tree.find_accepted_path({7, 11}) == P{7}));                      // root mismatch
    CHECK((tree.find_accepted_path({10}) == P{10}));
    CHECK((tree.find_accepted_path({10, 11}) == P{10, 11}));
    using N = std::vector<int>;
    CHECK((tree.find_accepted_nodes({10, 11, 14, 16}) == N{0, 1, 4, 6}));
    CHECK((tree.find_accepted_nodes({10, 12, 15, 99}) == N{0, 2, 5}));
    CHECK((tree.find_accepted_nodes({10, 11, 99, 5}) == N{0, 1}));   // the closing token has no node
    CHECK(tree.find_accepted_nodes({7, 11}).empty());                 // the root was replaced
    CHECK((tree.find_accepted_nodes({10}) == N{0}));
    tree.clear();
    CHECK(tree.size() == 0 && tree.max_depth() == 0);
}

TEST_CASE(factory_knows_only_hip) {
    CHECK(create_backend(BackendType::CPU) == nullptr);
    CHECK(create_backend(BackendType::Metal) == nullptr);
    auto hip = create_backend(BackendType::HIP);
    REQUIRE(hip != nullptr);
    CHECK(hip->get_type() == BackendType::HIP && !hip->is_initialized());
    CHECK_CODE(hip->create_buffer(BufferDesc::device(16)), ErrorCode::BackendNotInitialized);
    CHECK(hip_device_pointer(nullptr, BufferHandle{1}) == nullptr);
    HostMemoryBackend be;
    CHECK(hip_device_pointer(&be, BufferHandle{1}) == nullptr);
}

extern "C" void go_rope_table(float* cos_out, float* sin_out, int max_seq_len, int head_dim, float theta);

TEST_CASE(rope_cache_tables_and_checks) {
    // tests/test_llm.cpp:14-63 of the reference: sizes, position 0, position 1
    RoPECache cache;
    CHECK(!cache.is_initialized());
    cache.initialize(2048, 64, 10000.0f);
    CHECK(cache.is_initialized());
    CHECK(cache.cos_cache().size() == size_t(2048) * 32);
    CHECK(cache.sin_cache().size() == size_t(2048) * 32);
    RoPECache small;
    small.initialize(1024, 8, 10000.0f);
    for (int i = 0; i < 4; ++i) {
        CHECK(std::fabs(small.cos_cache()[i] - 1.0f) <= 1e-5f);
        CHECK(std::fabs(small.sin_cache()[i]) <= 1e-5f);
        const float angle = 1.0f / std::pow(10000.0f, static_cast<float>(2 * i) / 8);
        CHECK(std::fabs(small.cos_cache()[4 + i] - std::cos(angle)) <= 1e-5f);
        CHECK(std::fabs(small.sin_cache()[4 + i] - std::sin(angle)) <= 1e-5f);
    }
    // same bits as the oracle's table
    std::vector<float> c(size_t(1024) * 4), s(c.size());
    go_rope_table(c.data(), s.data(), 1024, 8, 10000.0f);
    CHECK(small.cos_cache() == c);
    CHECK(small.sin_cache() == s);

    // argument checks come before anything touches a device
    HostMemoryBackend be;
    REQUIRE(be.initialize().ok());
    Tensor q = Tensor::allocate({1, 4, 2, 8}, DataType::FP32, &be).take();
    Tensor k = Tensor::allocate({1, 4, 1, 8}, DataType::FP32, &be).take();
    RoPECache none;
    CHECK_CODE(none.apply(q, k, 0, &be), ErrorCode::InvalidState);
    CHECK_CODE(small.apply(q, k, 1021, &be), ErrorCode::InvalidArgument);  // 1021 + 4 > 1024
    Tensor wrong_dim = Tensor::allocate({1, 4, 2, 16}, DataType::FP32, &be).take();
    CHECK_CODE(small.apply(wrong_dim, k, 0, &be), ErrorCode::ShapeMismatch);
    Tensor half_q = Tensor::allocate({1, 4, 2, 8}, DataType::FP16, &be).take();
    CHECK_CODE(small.apply(half_q, k, 0, &be), ErrorCode::DTypeMismatch);
    // a backend that is not the GPU is refused, never computed on the host
    CHECK_CODE(small.apply(q, k, 0, &be), ErrorCode::BackendNotSupported);
}

TEST_CASE(commit_tree_path_checks) {
    HostMemoryBackend be;
    REQUIRE(be.initialize().ok());
    PagedKVConfig cfg;
    cfg.block_size = 16;
    cfg.num_blocks = 8;
    cfg.num_layers = 1;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 128;
    BlockManager mgr;
    REQUIRE(mgr.initialize(cfg, &be).ok());
    PagedKVCache seq(&mgr);
    PagedKVCache orphan;
    Tensor kt = Tensor::allocate({2, 6, 128}, DataType::FP16, &be).take();
    std::vector<Tensor> trees{kt};
    const int nodes[2] = {0, 3}, bad_nodes[1] = {6};
    CHECK_CODE(commit_tree_path(orphan, 0, nodes, trees, trees, &be), ErrorCode::InvalidState);
    CHECK_CODE(commit_tree_path(seq, 0, nodes, {}, {}, &be), ErrorCode::InvalidArgument);
    CHECK_CODE(commit_tree_path(seq, 0, nodes, trees, trees, &be), ErrorCode::BackendNotSupported);
    (void)bad_nodes;
}

TEST_CASE(paged_decode_batch_checks) {
    HostMemoryBackend be;
    REQUIRE(be.initialize().ok());
    PagedDecodeBatch step;
    PagedKVPool empty;
    CHECK_CODE(step.initialize(nullptr, 4, 4, &be), ErrorCode::InvalidState);
    CHECK_CODE(step.initialize(&empty, 4, 4, &be), ErrorCode::InvalidState);
    ModelConfig cfg;
    cfg.num_layers = 1;
    cfg.num_heads = 4;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 128;
    PagedKVPool pool;
    REQUIRE(pool.initialize(cfg, 2, 64, 16, &be).ok());
    CHECK_CODE(step.initialize(&pool, 0, 4, &be), ErrorCode::InvalidArgument);
    // never computed on a backend that is not the GPU
    CHECK_CODE(step.initialize(&pool, 4, 4, &be), ErrorCode::BackendNotSupported);
    const int slots[1] = {0};
    CHECK_CODE(step.begin_step(std::span<const int>(slots, 1)), ErrorCode::InvalidState);
}

// The branch order of TransformerModel::attention_gpu (src/llm/transformer.mm:4837-5051).
TEST_CASE(attention_gpu_dispatch_decision) {
    AttentionRequest r;
    r.total_tokens = 1;
    r.start_pos = 40;
    r.paged_attention = true;
    r.has_gpu_cache = true;
    r.gpu_cache_len = 12;      // paged attention wins whatever the contiguous GPU cache holds (:4850)
    auto path = select_attention_path(r);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::PagedDecode);

    r.paged_attention = false;
    r.gpu_cache_max_seq_len = 4096;
    r.gpu_cache_len = 40;      // in sync: the full GPU decode (:4878)
    path = select_attention_path(r);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::FullDecode);

    r.gpu_cache_len = 30;      // behind the host cache, which covers start_pos: sync, then decode (:4890)
    r.host_cache_len = 40;
    path = select_attention_path(r);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::SyncThenFullDecode);
    r.host_cache_len = 35;     // the host cache does not cover it either: the reference goes to its CPU path
    CHECK_CODE(select_attention_path(r), ErrorCode::InvalidState);
    r.host_cache_len = -1;
    r.gpu_cache_len = 50;      // ahead: "something is wrong" (:4911)
    CHECK_CODE(select_attention_path(r), ErrorCode::InvalidState);

    // the offload branch comes before the decode branches and leaves the GPU (:4861-4872)
    r.kv_cache_offload = true;
    r.gpu_cache_max_seq_len = 40;
    r.gpu_cache_len = 40;
    CHECK_CODE(select_attention_path(r), ErrorCode::BackendNotSupported);
    r.gpu_cache_max_seq_len = 41;
    path = select_attention_path(r);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::FullDecode);
    r.paged_attention = true;  // ... but after the paged branch
    r.gpu_cache_max_seq_len = 40;
    path = select_attention_path(r);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::PagedDecode);

    // several tokens: the GPU prefill only from position 0 and only with a GPU cache (:4915)
    AttentionRequest p;
    p.total_tokens = 300;
    p.has_gpu_cache = true;
    p.gpu_cache_max_seq_len = 4096;
    path = select_attention_path(p);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::Prefill);
    p.paged_attention = true;  // the paged branch is for single tokens only
    path = select_attention_path(p);
    REQUIRE(path.ok());
    CHECK(path.value() == AttentionPath::Prefill);
    p.start_pos = 64;
    CHECK_CODE(select_attention_path(p), ErrorCode::InvalidState);
    p.start_pos = 0;
    p.has_gpu_cache = false;
    CHECK_CODE(select_attention_path(p), ErrorCode::InvalidState);
    p.total_tokens = 0;
    CHECK_CODE(select_attention_path(p), ErrorCode::InvalidArgument);
}

TEST_CASE(tree_verify_checks) {
    HostMemoryBackend be;
    REQUIRE(be.initialize().ok());
    TreeVerify verify;
    const int parents[3] = {-1, 0, 0};
    CHECK_CODE(verify.begin(parents), ErrorCode::InvalidState);
    CHECK_CODE(verify.initialize(nullptr, 4, 8, &be), ErrorCode::InvalidState);
    PagedKVConfig cfg;
    cfg.block_size = 16;
    cfg.num_blocks = 4;
    cfg.num_layers = 1;
    cfg.num_kv_heads = 2;
    cfg.head_dim = 128;
    BlockManager mgr;
    REQUIRE(mgr.initialize(cfg, &be).ok());
    PagedKVCache seq(&mgr);
    CHECK_CODE(verify.initialize(&seq, 0, 8, &be), ErrorCode::InvalidArgument);
    // never computed on a backend that is not the GPU
    CHECK_CODE(verify.initialize(&seq, 4, 8, &be), ErrorCode::BackendNotSupported);
}

int main(int argc, char** argv) { return hosttest::run_all(argc, argv); }
