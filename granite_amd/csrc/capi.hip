// C ABI of libgranite_hip.so: device lifecycle, memory, timing, and the
// argument checking in front of the kernel launchers.  This and the kernel
// files are the only code that includes hip_runtime.h; everything above talks
// to the functions declared in granite_hip.h.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "common.h"

// Scratch memory of granite_hip_decode_attention_static, the entry point for callers
// that cannot allocate.  One copy per device, held until the process ends.  In host code
// this name is only a handle for hipGetSymbolAddress: the address kernels and copies use
// is the one resolved per device in granite_hip_init.
static constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace ghip {

namespace {
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};  // device address of `scratch`, per device
}  // namespace

Context& ctx() {
    static Context c;
    return c;
}

int ensure_workspace(size_t bytes) {
    Context& c = ctx();
    if (bytes <= c.workspace_bytes) return GRANITE_HIP_OK;
    // Earlier launches, on this stream or on one the caller used before
    // granite_hip_set_stream, may still use the old buffer.
    GHIP_CHECK(hipDeviceSynchronize());
    if (c.workspace) GHIP_CHECK(hipFree(c.workspace));
    c.workspace = nullptr;
    c.workspace_bytes = 0;
    size_t want = bytes + bytes / 4;
    want = (want + 255) & ~size_t(255);
    hipError_t e = hipMalloc(&c.workspace, want);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return GRANITE_HIP_ENOMEM;
    }
    c.workspace_bytes = want;
    return GRANITE_HIP_OK;
}

int take_scratch(const ScratchSource& src, size_t need, void** ws) {
    *ws = nullptr;
    if (src.query) {
        *src.query = need;
        return GRANITE_HIP_OK;
    }
    if (src.fixed) {
        if (need > src.fixed_bytes) return GRANITE_HIP_ESCRATCH;
        if (reinterpret_cast<uintptr_t>(src.fixed) & 255) return GRANITE_HIP_EINVAL;
        *ws = src.fixed;
        return GRANITE_HIP_OK;
    }
    int rc = ensure_workspace(need);
    if (rc != GRANITE_HIP_OK) return rc;
    *ws = ctx().workspace;
    return GRANITE_HIP_OK;
}

namespace {
struct PendingTiming {
    const char* name;
    hipEvent_t start, stop;
};
struct TimingState {
    bool enabled = false;
    bool suppressed = false;  // inside an entry point that must not create events
    std::vector<PendingTiming> pending;
    std::vector<hipEvent_t> free_events;
    std::map<std::string, std::pair<double, uint64_t>> stats;
};
TimingState& timing() {
    static TimingState t;
    return t;
}
hipEvent_t take_event() {
    TimingState& t = timing();
    if (!t.free_events.empty()) {
        hipEvent_t e = t.free_events.back();
        t.free_events.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}
// Waits for the stream and folds every finished (start, stop) pair into the table.
void resolve_timings() {
    TimingState& t = timing();
    if (t.pending.empty()) return;
    (void)hipStreamSynchronize(ctx().stream);
    for (const PendingTiming& p : t.pending) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
            auto& slot = t.stats[p.name];
            slot.first += ms;
            slot.second += 1;
        }
        t.free_events.push_back(p.start);
        t.free_events.push_back(p.stop);
    }
    t.pending.clear();
}
}  // namespace

TimingSuppressed::TimingSuppressed() : was_(timing().suppressed) { timing().suppressed = true; }
TimingSuppressed::~TimingSuppressed() { timing().suppressed = was_; }

KernelTimerScope::KernelTimerScope(const char* name) : name_(name) {
    if (!timing().enabled || timing().suppressed) return;
    start_ = take_event();
    if (start_) (void)hipEventRecord(start_, ctx().stream);
}

KernelTimerScope::~KernelTimerScope() {
    if (!start_) return;
    hipEvent_t stop = take_event();
    if (!stop) {
        timing().free_events.push_back(start_);
        return;
    }
    (void)hipEventRecord(stop, ctx().stream);
    timing().pending.push_back({name_, start_, stop});
}

}  // namespace ghip

using ghip::ctx;

extern "C" {

const char* granite_hip_version(void) { return "granite-hip 0.1 (gfx950)"; }

const char* granite_hip_error_string(int code) {
    switch (code) {
        case GRANITE_HIP_OK: return "ok";
        case GRANITE_HIP_EINVAL: return "InvalidArgument";
        case GRANITE_HIP_ENOTINIT: return "BackendNotInitialized";
        case GRANITE_HIP_ENOMEM: return "AllocationFailed";
        case GRANITE_HIP_EUNSUPPORTED: return "NotImplemented";
        case GRANITE_HIP_ENULL: return "NullPointer";
        case GRANITE_HIP_EOVERFLOW: return "InvalidArgument: KV cache overflow";
        case GRANITE_HIP_ESCRATCH: return "InvalidArgument: the launch needs more scratch memory than the buffer given holds";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error";
}

int granite_hip_init(int device) {
    ghip::Context& c = ctx();
    if (c.initialized) return c.device == device ? GRANITE_HIP_OK : GRANITE_HIP_EINVAL;
    int count = 0;
    GHIP_CHECK(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return GRANITE_HIP_EINVAL;
    GHIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    GHIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        std::fprintf(stderr, "granite_hip: device %d is %s; this library holds gfx950 code only\n",
                     device, prop.gcnArchName);
        return GRANITE_HIP_EUNSUPPORTED;
    }
    if (device >= ghip::kMaxDevices) return GRANITE_HIP_EINVAL;
    if (!ghip::g_static_scratch[device]) {
        // every device holds its own copy of the array at its own address
        void* ptr = nullptr;
        GHIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr || (reinterpret_cast<uintptr_t>(ptr) & 255)) return GRANITE_HIP_EINVAL;
        ghip::g_static_scratch[device] = ptr;
    }
    GHIP_CHECK(hipStreamCreateWithFlags(&c.own_stream, hipStreamNonBlocking));
    c.stream = c.own_stream;
    c.device = device;
    c.compute_units = prop.multiProcessorCount;
    c.initialized = true;
    return GRANITE_HIP_OK;
}

int granite_hip_shutdown(void) {
    ghip::Context& c = ctx();
    if (!c.initialized) return GRANITE_HIP_OK;
    (void)hipStreamSynchronize(c.stream);
    if (c.workspace) (void)hipFree(c.workspace);
    c.workspace = nullptr;
    c.workspace_bytes = 0;
    ghip::resolve_timings();
    for (hipEvent_t e : ghip::timing().free_events) (void)hipEventDestroy(e);
    ghip::timing().free_events.clear();
    ghip::timing().stats.clear();
    ghip::timing().enabled = false;
    if (c.own_stream) (void)hipStreamDestroy(c.own_stream);
    c.own_stream = nullptr;
    c.stream = nullptr;
    c.initialized = false;
    return GRANITE_HIP_OK;
}

int granite_hip_is_initialized(void) { return ctx().initialized ? 1 : 0; }

int granite_hip_get_device_info(granite_hip_device_info* info) {
    GHIP_REQUIRE_INIT();
    if (!info) return GRANITE_HIP_ENULL;
    hipDeviceProp_t prop;
    GHIP_CHECK(hipGetDeviceProperties(&prop, ctx().device));
    std::memset(info, 0, sizeof(*info));
    std::snprintf(info->name, sizeof(info->name), "%s", prop.name);
    std::snprintf(info->arch, sizeof(info->arch), "%s", prop.gcnArchName);
    info->total_memory = prop.totalGlobalMem;
    info->max_buffer_size = prop.totalGlobalMem;
    info->shared_memory_per_block = prop.sharedMemPerBlock;
    info->max_threads_per_block = prop.maxThreadsPerBlock;
    info->wavefront_size = prop.warpSize;
    info->compute_units = prop.multiProcessorCount;
    info->clock_khz = prop.clockRate;
    return GRANITE_HIP_OK;
}

int granite_hip_malloc(void** ptr, size_t bytes, int memory_kind) {
    GHIP_REQUIRE_INIT();
    if (!ptr) return GRANITE_HIP_ENULL;
    *ptr = nullptr;
    if (bytes == 0) return GRANITE_HIP_EINVAL;
    hipError_t e;
    if (memory_kind == GRANITE_HIP_MEM_SHARED)
        e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
    else if (memory_kind == GRANITE_HIP_MEM_DEVICE || memory_kind == GRANITE_HIP_MEM_MANAGED)
        e = hipMalloc(ptr, bytes);
    else
        return GRANITE_HIP_EINVAL;
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *ptr = nullptr;
        return e == hipErrorOutOfMemory ? GRANITE_HIP_ENOMEM : static_cast<int>(e);
    }
    return GRANITE_HIP_OK;
}

int granite_hip_free(void* ptr, int memory_kind) {
    GHIP_REQUIRE_INIT();
    if (!ptr) return GRANITE_HIP_OK;
    if (memory_kind == GRANITE_HIP_MEM_SHARED) GHIP_CHECK(hipHostFree(ptr));
    else GHIP_CHECK(hipFree(ptr));
    return GRANITE_HIP_OK;
}

int granite_hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    GHIP_REQUIRE_INIT();
    if (bytes == 0) return GRANITE_HIP_OK;
    if (!dst || !src) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx().stream));
    GHIP_CHECK(hipStreamSynchronize(ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    GHIP_REQUIRE_INIT();
    if (bytes == 0) return GRANITE_HIP_OK;
    if (!dst || !src) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx().stream));
    GHIP_CHECK(hipStreamSynchronize(ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    GHIP_REQUIRE_INIT();
    if (bytes == 0) return GRANITE_HIP_OK;
    if (!dst || !src) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_memset(void* dst, int value, size_t bytes) {
    GHIP_REQUIRE_INIT();
    if (bytes == 0) return GRANITE_HIP_OK;
    if (!dst) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipMemsetAsync(dst, value, bytes, ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_sync(void) {
    GHIP_REQUIRE_INIT();
    GHIP_CHECK(hipStreamSynchronize(ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_set_stream(void* stream) {
    GHIP_REQUIRE_INIT();
    ghip::Context& c = ctx();
    hipStream_t next = stream ? static_cast<hipStream_t>(stream) : c.own_stream;
    if (next == c.stream) return GRANITE_HIP_OK;
    // All launches share one scratch buffer: whatever is still queued on the old stream
    // has to finish before a launch on the new one may overwrite its partials.
    ghip::resolve_timings();
    hipEvent_t done = nullptr;
    GHIP_CHECK(hipEventCreateWithFlags(&done, hipEventDisableTiming));
    hipError_t e = hipEventRecord(done, c.stream);
    if (e == hipSuccess) e = hipStreamWaitEvent(next, done, 0);
    (void)hipEventDestroy(done);  // released once the recorded work has completed
    if (e != hipSuccess) return static_cast<int>(e);
    c.stream = next;
    return GRANITE_HIP_OK;
}

void* granite_hip_get_stream(void) { return ctx().initialized ? ctx().stream : nullptr; }

int granite_hip_event_create(void** event) {
    GHIP_REQUIRE_INIT();
    if (!event) return GRANITE_HIP_ENULL;
    hipEvent_t e;
    GHIP_CHECK(hipEventCreate(&e));
    *event = e;
    return GRANITE_HIP_OK;
}

int granite_hip_event_destroy(void* event) {
    GHIP_REQUIRE_INIT();
    if (!event) return GRANITE_HIP_OK;
    GHIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return GRANITE_HIP_OK;
}

int granite_hip_event_record(void* event) {
    GHIP_REQUIRE_INIT();
    if (!event) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), ctx().stream));
    return GRANITE_HIP_OK;
}

int granite_hip_event_synchronize(void* event) {
    GHIP_REQUIRE_INIT();
    if (!event) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return GRANITE_HIP_OK;
}

int granite_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    GHIP_REQUIRE_INIT();
    if (!start || !stop || !ms) return GRANITE_HIP_ENULL;
    GHIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start),
                                   static_cast<hipEvent_t>(stop)));
    return GRANITE_HIP_OK;
}

int granite_hip_kv_commit_accepted(const void* k_tree, const void* v_tree, int src_dtype,
                                   int64_t src_tok_stride, int64_t src_head_stride,
                                   uint32_t num_nodes, const int32_t* accepted_nodes,
                                   uint32_t num_accepted, void* k_cache, void* v_cache,
                                   const int32_t* block_table, uint32_t num_kv_heads,
                                   uint32_t head_dim, uint32_t start_pos, uint32_t block_size,
                                   uint32_t max_seq_len, int rounding) {
    GHIP_REQUIRE_INIT();
    if (num_accepted == 0) return GRANITE_HIP_OK;
    if (!accepted_nodes) return GRANITE_HIP_ENULL;
    if (num_nodes == 0) return GRANITE_HIP_EINVAL;
    if (block_table)
        return ghip::launch_kv_append_paged(k_tree, v_tree, src_dtype, src_tok_stride, src_head_stride,
                                            k_cache, v_cache, block_table, num_kv_heads, head_dim,
                                            start_pos, num_accepted, block_size, rounding,
                                            accepted_nodes, num_nodes);
    return ghip::launch_kv_append_contig(k_cache, v_cache, k_tree, v_tree, src_dtype, src_tok_stride,
                                         src_head_stride, num_kv_heads, head_dim, start_pos,
                                         num_accepted, max_seq_len, rounding, accepted_nodes, num_nodes);
}

// ---- RoPE (+ append) -----------------------------------------------------

int granite_hip_rope_append(const granite_hip_rope_args* args) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    return ghip::launch_rope_append(*args);
}

int granite_hip_rope_multihead(void* q, void* k, uint32_t num_heads_q, uint32_t num_heads_k,
                               uint32_t seq_len, uint32_t head_dim, uint32_t start_pos,
                               float freq_base) {
    GHIP_REQUIRE_INIT();
    granite_hip_rope_args a{};
    a.q = q;
    a.k = k;
    a.num_heads_q = num_heads_q;
    a.num_heads_k = num_heads_k;
    a.seq_len = seq_len;
    a.head_dim = head_dim;
    a.start_pos = start_pos;
    a.freq_base = freq_base;
    a.write_k_back = 1;
    a.rounding = GRANITE_HIP_ROUND_TRUNCATE;
    return ghip::launch_rope_append(a);
}

size_t granite_hip_workspace_bytes(void) { return ctx().workspace_bytes; }

int granite_hip_reserve_workspace(size_t bytes) {
    GHIP_REQUIRE_INIT();
    return ghip::ensure_workspace(bytes);
}

int granite_hip_decode_workspace_required(const granite_hip_decode_args* args, size_t* bytes) {
    GHIP_REQUIRE_INIT();
    if (!args || !bytes) return GRANITE_HIP_ENULL;
    ghip::ScratchSource src;
    src.query = bytes;
    return ghip::launch_decode(*args, src);
}

int granite_hip_attention_workspace_required(const granite_hip_attention_args* args, size_t* bytes) {
    GHIP_REQUIRE_INIT();
    if (!args || !bytes) return GRANITE_HIP_ENULL;
    ghip::ScratchSource src;
    src.query = bytes;
    return ghip::launch_attention(*args, src);
}

int granite_hip_decode_attention_ws(const granite_hip_decode_args* args, void* workspace,
                                    size_t workspace_bytes) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    if (!workspace) return ghip::launch_decode(*args);
    ghip::ScratchSource src;
    src.fixed = workspace;
    src.fixed_bytes = workspace_bytes;
    return ghip::launch_decode(*args, src);
}

size_t granite_hip_static_scratch_bytes(void) { return kStaticScratchBytes; }

int granite_hip_decode_attention_static(const granite_hip_decode_args* args) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    ghip::ScratchSource src;
    src.fixed = ghip::g_static_scratch[ctx().device];
    src.fixed_bytes = kStaticScratchBytes;
    if (!src.fixed) return GRANITE_HIP_ENOTINIT;
    // no events either: per-kernel timing creates them on demand
    ghip::TimingSuppressed quiet;
    return ghip::launch_decode(*args, src);
}

int granite_hip_attention_ws(const granite_hip_attention_args* args, void* workspace,
                             size_t workspace_bytes) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    if (!workspace) return ghip::launch_attention(*args);
    ghip::ScratchSource src;
    src.fixed = workspace;
    src.fixed_bytes = workspace_bytes;
    return ghip::launch_attention(*args, src);
}

int granite_hip_enable_kernel_timing(int enable) {
    GHIP_REQUIRE_INIT();
    ghip::resolve_timings();
    ghip::timing().enabled = enable != 0;
    return GRANITE_HIP_OK;
}

int granite_hip_reset_kernel_timing(void) {
    GHIP_REQUIRE_INIT();
    ghip::resolve_timings();
    ghip::timing().stats.clear();
    return GRANITE_HIP_OK;
}

int granite_hip_get_kernel_timing(const char* kernel_name, double* total_ms,
                                  uint64_t* dispatches) {
    GHIP_REQUIRE_INIT();
    if (!kernel_name || !total_ms || !dispatches) return GRANITE_HIP_ENULL;
    ghip::resolve_timings();
    auto it = ghip::timing().stats.find(kernel_name);
    if (it == ghip::timing().stats.end()) {
        *total_ms = 0.0;
        *dispatches = 0;
        return GRANITE_HIP_OK;
    }
    *total_ms = it->second.first;
    *dispatches = it->second.second;
    return GRANITE_HIP_OK;
}

int granite_hip_kernel_timing_names(char* buffer, size_t buffer_bytes) {
    GHIP_REQUIRE_INIT();
    if (!buffer || buffer_bytes == 0) return GRANITE_HIP_ENULL;
    ghip::resolve_timings();
    std::string all;
    for (const auto& kv : ghip::timing().stats) {
        if (!all.empty()) all += ',';
        all += kv.first;
    }
    if (all.size() + 1 > buffer_bytes) return GRANITE_HIP_EINVAL;
    std::memcpy(buffer, all.c_str(), all.size() + 1);
    return GRANITE_HIP_OK;
}

// ---- KV append / gather -------------------------------------------------

int granite_hip_kv_cache_append(void* cache_k, void* cache_v, const void* new_k,
                                const void* new_v, uint32_t num_kv_heads, uint32_t head_dim,
                                uint32_t current_len, uint32_t new_len, uint32_t max_seq_len) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_kv_append_contig(cache_k, cache_v, new_k, new_v, GRANITE_HIP_F32,
                                         int64_t(num_kv_heads) * head_dim, head_dim, num_kv_heads,
                                         head_dim, current_len, new_len, max_seq_len,
                                         GRANITE_HIP_ROUND_TRUNCATE);
}

int granite_hip_kv_cache_append_ex(void* cache_k, void* cache_v, const void* new_k,
                                   const void* new_v, int src_dtype, int64_t src_tok_stride,
                                   int64_t src_head_stride, uint32_t num_kv_heads,
                                   uint32_t head_dim, uint32_t current_len, uint32_t new_len,
                                   uint32_t max_seq_len, int rounding) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_kv_append_contig(cache_k, cache_v, new_k, new_v, src_dtype,
                                         src_tok_stride, src_head_stride, num_kv_heads, head_dim,
                                         current_len, new_len, max_seq_len, rounding);
}

int granite_hip_paged_kv_cache_append(const void* new_k, const void* new_v, void* k_cache,
                                      void* v_cache, const int32_t* block_table,
                                      uint32_t num_kv_heads, uint32_t head_dim,
                                      uint32_t start_pos, uint32_t new_len, uint32_t block_size) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_kv_append_paged(new_k, new_v, GRANITE_HIP_F32, head_dim,
                                        int64_t(new_len) * head_dim, k_cache, v_cache, block_table,
                                        num_kv_heads, head_dim, start_pos, new_len, block_size,
                                        GRANITE_HIP_ROUND_TRUNCATE);
}

int granite_hip_paged_kv_cache_append_ex(const void* new_k, const void* new_v, int src_dtype,
                                         int64_t src_tok_stride, int64_t src_head_stride,
                                         void* k_cache, void* v_cache,
                                         const int32_t* block_table, uint32_t num_kv_heads,
                                         uint32_t head_dim, uint32_t start_pos,
                                         uint32_t new_len, uint32_t block_size, int rounding,
                                         uint32_t max_blocks) {
    GHIP_REQUIRE_INIT();
    if (max_blocks > 0 && block_size > 0 &&
        (uint64_t(start_pos) + new_len + block_size - 1) / block_size > max_blocks)
        return GRANITE_HIP_EOVERFLOW;
    return ghip::launch_kv_append_paged(new_k, new_v, src_dtype, src_tok_stride, src_head_stride,
                                        k_cache, v_cache, block_table, num_kv_heads, head_dim,
                                        start_pos, new_len, block_size, rounding);
}

int granite_hip_paged_kv_gather(void* dst_k, void* dst_v, const void* k_cache,
                                const void* v_cache, const int32_t* block_table,
                                uint32_t num_kv_heads, uint32_t head_dim, uint32_t len,
                                uint32_t block_size, uint32_t max_seq_len) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_kv_gather_paged(dst_k, dst_v, k_cache, v_cache, block_table, num_kv_heads,
                                        head_dim, len, block_size, max_seq_len);
}

int granite_hip_copy_rows(void* dst, int64_t dst_row_bytes, const void* src, int64_t src_row_bytes,
                          uint64_t rows, uint32_t copy_bytes, uint32_t fill_bytes) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_copy_rows(dst, dst_row_bytes, src, src_row_bytes, rows, copy_bytes, fill_bytes);
}

// ---- projections on Q4_K weights ------------------------------------------------

int granite_hip_fused_qkv_matvec_q4k_batched(const void* x, int64_t x_stride, const void* wq,
                                             const void* wk, const void* wv, void* yq, void* yk,
                                             void* yv, int64_t yq_stride, int64_t ykv_stride,
                                             uint32_t K, uint32_t Nq, uint32_t Nkv, uint32_t batch) {
    GHIP_REQUIRE_INIT();
    const void* const w[3] = {wq, wk, wv};
    void* const y[3] = {yq, yk, yv};
    const int64_t ys[3] = {yq_stride, ykv_stride, ykv_stride};
    const uint32_t n[3] = {Nq, Nkv, Nkv};
    return ghip::launch_matvec_q4k(x, x_stride, w, y, ys, n, K, batch);
}

int granite_hip_fused_qkv_matvec_q4k(const void* x, const void* wq, const void* wk, const void* wv,
                                     void* yq, void* yk, void* yv, uint32_t K, uint32_t Nq,
                                     uint32_t Nkv) {
    return granite_hip_fused_qkv_matvec_q4k_batched(x, K, wq, wk, wv, yq, yk, yv, Nq, Nkv, K, Nq, Nkv, 1);
}

int granite_hip_matvec_q4k_batched(const void* x, int64_t x_stride, const void* w, void* y,
                                   int64_t y_stride, uint32_t K, uint32_t N, uint32_t batch) {
    GHIP_REQUIRE_INIT();
    const void* const ws[3] = {w, nullptr, nullptr};
    void* const ys[3] = {y, nullptr, nullptr};
    const int64_t strides[3] = {y_stride, 0, 0};
    const uint32_t n[3] = {N, 0, 0};
    return ghip::launch_matvec_q4k(x, x_stride, ws, ys, strides, n, K, batch);
}

size_t granite_hip_q4k_workspace_required(uint32_t K, uint64_t rows, uint32_t batch) {
    return ghip::matvec_q4k_scratch_bytes(K, rows, batch);
}

int granite_hip_matvec_q4k(const void* x, const void* w, void* y, uint32_t K, uint32_t N) {
    return granite_hip_matvec_q4k_batched(x, K, w, y, N, K, N, 1);
}

// ---- attention ------------------------------------------------------------

int granite_hip_decode_attention(const granite_hip_decode_args* args) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    return ghip::launch_decode(*args);
}

int granite_hip_attention(const granite_hip_attention_args* args) {
    GHIP_REQUIRE_INIT();
    if (!args) return GRANITE_HIP_ENULL;
    return ghip::launch_attention(*args);
}

int granite_hip_build_tree_mask(const int32_t* parent_indices, uint32_t* mask_words,
                                uint32_t num_nodes) {
    GHIP_REQUIRE_INIT();
    return ghip::launch_tree_mask(parent_indices, mask_words, num_nodes);
}

int granite_hip_multihead_attention(const void* q, const void* k, const void* v, void* out,
                                    uint32_t num_heads, uint32_t num_kv_heads, uint32_t seq_q,
                                    uint32_t seq_kv, uint32_t head_dim, float scale,
                                    uint32_t max_seq) {
    GHIP_REQUIRE_INIT();
    if (max_seq == 0) max_seq = seq_kv;  // metal_compute.mm:2259-2260
    if (seq_kv == 0 || seq_kv > max_seq) return GRANITE_HIP_EINVAL;
    if (seq_q == 1) {
        // Decode: one workgroup set over the contiguous cache, length fixed by the caller.
        granite_hip_decode_args d{};
        d.q = q;
        d.q_dtype = GRANITE_HIP_F32;
        d.k_cache = k;
        d.v_cache = v;
        d.out = out;
        d.batch_size = 1;
        d.num_heads = num_heads;
        d.num_kv_heads = num_kv_heads;
        d.head_dim = head_dim;
        d.max_seq = max_seq;
        d.fixed_seq_len = seq_kv;
        d.scale = scale;
        return ghip::launch_decode(d);
    }
    granite_hip_attention_args a{};
    a.q = q;
    a.q_dtype = GRANITE_HIP_F32;
    a.q_tok_stride = int64_t(num_heads) * head_dim;
    a.q_head_stride = head_dim;
    a.out = out;
    a.out_dtype = GRANITE_HIP_F32;
    a.out_tok_stride = a.q_tok_stride;
    a.out_head_stride = head_dim;
    a.k_cache = k;
    a.v_cache = v;
    a.max_seq = max_seq;
    a.cache_len = seq_kv;
    a.mask_mode = GRANITE_HIP_MASK_CAUSAL;
    a.start_pos = 0;  // the reference passes 0 to its prefill kernel (metal_compute.mm:2352)
    a.seq_q = seq_q;
    a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads;
    a.head_dim = head_dim;
    a.scale = scale;
    return ghip::launch_attention(a);
}

int granite_hip_attention_tree(const void* q, const void* k_cache, const void* v_cache,
                               const void* k_tree, const void* v_tree,
                               const int32_t* parent_indices, void* out, uint32_t num_heads,
                               uint32_t num_kv_heads, uint32_t num_nodes, uint32_t cache_len,
                               uint32_t head_dim, float scale) {
    GHIP_REQUIRE_INIT();
    granite_hip_attention_args a{};
    a.q = q;
    a.q_dtype = GRANITE_HIP_F32;
    a.q_tok_stride = head_dim;  // [num_heads, num_nodes, D]
    a.q_head_stride = int64_t(num_nodes) * head_dim;
    a.out = out;
    a.out_dtype = GRANITE_HIP_F32;
    a.out_tok_stride = head_dim;
    a.out_head_stride = a.q_head_stride;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.max_seq = cache_len;
    a.cache_len = cache_len;
    a.k_extra = k_tree;
    a.v_extra = v_tree;
    a.extra_len = num_nodes;
    a.parents = parent_indices;
    a.mask_mode = GRANITE_HIP_MASK_TREE;
    a.seq_q = num_nodes;
    a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads;
    a.head_dim = head_dim;
    a.scale = scale;
    return ghip::launch_attention(a);
}

int granite_hip_paged_attention_decode(const void* q, const void* k_cache, const void* v_cache,
                                       const int32_t* block_table, void* out,
                                       uint32_t num_heads, uint32_t num_kv_heads,
                                       uint32_t seq_len, uint32_t head_dim,
                                       uint32_t block_size, float scale) {
    GHIP_REQUIRE_INIT();
    if (!block_table) return GRANITE_HIP_ENULL;
    if (seq_len == 0 || block_size == 0) return GRANITE_HIP_EINVAL;
    granite_hip_decode_args d{};
    d.q = q;
    d.q_dtype = GRANITE_HIP_F32;
    d.k_cache = k_cache;
    d.v_cache = v_cache;
    d.block_tables = block_table;
    d.out = out;
    d.batch_size = 1;
    d.num_heads = num_heads;
    d.num_kv_heads = num_kv_heads;
    d.head_dim = head_dim;
    d.block_size = block_size;
    d.max_blocks_per_seq = (seq_len + block_size - 1) / block_size;
    d.fixed_seq_len = seq_len;
    d.scale = scale;
    return ghip::launch_decode(d);
}

int granite_hip_batched_paged_attention_decode(const void* q, const void* k_cache,
                                               const void* v_cache,
                                               const int32_t* block_tables,
                                               const int32_t* seq_lens, void* out,
                                               uint32_t batch_size, uint32_t num_heads,
                                               uint32_t num_kv_heads, uint32_t head_dim,
                                               uint32_t block_size,
                                               uint32_t max_blocks_per_seq, float scale) {
    GHIP_REQUIRE_INIT();
    if (!block_tables || !seq_lens) return GRANITE_HIP_ENULL;
    granite_hip_decode_args d{};
    d.q = q;
    d.q_dtype = GRANITE_HIP_F32;
    d.k_cache = k_cache;
    d.v_cache = v_cache;
    d.block_tables = block_tables;
    d.seq_lens = seq_lens;
    d.out = out;
    d.batch_size = batch_size;
    d.num_heads = num_heads;
    d.num_kv_heads = num_kv_heads;
    d.head_dim = head_dim;
    d.block_size = block_size;
    d.max_blocks_per_seq = max_blocks_per_seq;
    d.scale = scale;
    return ghip::launch_decode(d);
}

}  // extern "C"
