// ref_bind.cpp -- C entry points over the reference's own math_ops.cpp.
//
// TEST INFRASTRUCTURE.  Compiled only when the reference tree is present;
// the result lands in oracle/_ref/ and is used to check the restatement in
// granite_oracle.c (conversions, thread partitioning).  The reference source
// is compiled where it lies; nothing of it is copied here.
#include "math_ops.h"  // found through -I<reference>/src/llm

#include <atomic>
#include <cstdint>

extern "C" {

float ref_fp16_to_fp32(uint16_t h) { return granite::fp16_to_fp32(h); }
uint16_t ref_fp32_to_fp16(float f) { return granite::fp32_to_fp16(f); }
void ref_fp16_to_fp32_array(const uint16_t* src, float* dst, size_t n) {
    granite::fp16_to_fp32_array(src, dst, n);
}
size_t ref_get_num_threads() { return granite::get_num_threads(); }

// Runs the reference parallel_for and records which worker slot touched each
// index (owner[i] = chunk number), so the partition can be compared.
void ref_parallel_for_owner(size_t n, size_t num_threads, int32_t* owner) {
    size_t chunk = num_threads ? (n + num_threads - 1) / num_threads : n;
    granite::parallel_for(n, num_threads, [owner, chunk](size_t i) {
        owner[i] = chunk ? static_cast<int32_t>(i / chunk) : 0;
    });
}

// Counts calls; checks every index is visited exactly once.
size_t ref_parallel_for_count(size_t n, size_t num_threads, uint8_t* visited) {
    std::atomic<size_t> calls{0};
    granite::parallel_for(n, num_threads, [&calls, visited](size_t i) {
        visited[i]++;
        calls.fetch_add(1, std::memory_order_relaxed);
    });
    return calls.load();
}

// The reference's own projection routine (portable branch of matmul_transb).
void ref_matmul_transb_fp16(const float* A, const uint16_t* B_fp16, float* C, int M, int N, int K) {
    granite::matmul_transb_fp16(A, B_fp16, C, M, N, K);
}

}  // extern "C"
