// ref_bind.cpp -- C entry points over the reference's own math_ops.cpp.
//
// TEST INFRASTRUCTURE.  Compiled only when the reference tree is present;
// the result lands in oracle/_ref/ and is used to check the restatement in
// granite_oracle.c (conversions, thread partitioning).  The reference source
// is compiled where it lies; nothing of it is copied here.
#include "math_ops.h"  // found through -I<reference>/src/llm

#include <atomic>
#include <cstdint>
#include <map>
#include <thread>
#include <vector>

extern "C" {

float ref_fp16_to_fp32(uint16_t h) { return granite::fp16_to_fp32(h); }
uint16_t ref_fp32_to_fp16(float f) { return granite::fp32_to_fp16(f); }
void ref_fp16_to_fp32_array(const uint16_t* src, float* dst, size_t n) {
    granite::fp16_to_fp32_array(src, dst, n);
}
size_t ref_get_num_threads() { return granite::get_num_threads(); }

// Runs the reference parallel_for and records which thread ran each index, as the smallest
// index that thread ran (owner[i] == owner[j] iff one thread ran both; the threads of a call
// live until it joins them, so their ids are distinct).  That is the partition itself, not a
// formula for it.
void ref_parallel_for_owner(size_t n, size_t num_threads, int32_t* owner) {
    std::vector<std::thread::id> ran(n);
    granite::parallel_for(n, num_threads, [&ran](size_t i) { ran[i] = std::this_thread::get_id(); });
    std::map<std::thread::id, int32_t> first;
    for (size_t i = 0; i < n; i++) first.emplace(ran[i], static_cast<int32_t>(i));  // keeps the smallest
    for (size_t i = 0; i < n; i++) owner[i] = first[ran[i]];
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
