// The host side of the library (fbgemm_amd/csrc/c_api.cpp: plans, work-list cache, per-stream
// and per-thread scratch, the static scratch of the entry point that allocates nothing) driven
// on the CPU against the HIP stand-in of tests/cpp/hip_stub, built with
// -fsanitize=address,undefined. The sanitizers are the checker: a use after free, a double
// free, an overrun or a leak of "device" or host memory ends the program with a report. The
// scenarios are the lifetimes that have broken before: plan creation failing half-way, pruned-
// row mappings set twice, eviction from the work-list cache with entries a graph may hold,
// trimming, scratch handed from a host thread that has ended to a new one, split bags, the 8-bit
// pooled output, allocation failures at every point of a first forward.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/fbgemm_amd.h"
#include "../../include/fbgemm_amd_bench.h"

#define CHECK(cond)                                                         \
  do {                                                                      \
    if (!(cond)) {                                                          \
      printf("FAILED %s:%d: %s (%s)\n", __FILE__, __LINE__, #cond, fbgemm_amd_last_error()); \
      exit(1);                                                              \
    }                                                                       \
  } while (0)

namespace {

struct Problem {
  int32_t T;
  std::vector<int64_t> wo;
  std::vector<uint8_t> tys;
  std::vector<int32_t> D_offsets;
  int64_t bytes;
};

// int4 / int8 / fp16 / int2 tables of a few rows each (sizes only: no kernel reads them here)
Problem make_problem(int32_t T) {
  Problem p;
  p.T = T;
  const int32_t Ds[4] = {64, 128, 256, 32};
  const uint8_t tys[4] = {3, 2, 1, 4};
  int64_t off = 0;
  p.D_offsets.push_back(0);
  for (int t = 0; t < T; ++t) {
    p.wo.push_back(off);
    p.tys.push_back(tys[t % 4]);
    p.D_offsets.push_back(p.D_offsets.back() + Ds[t % 4]);
    const int64_t row = fbgemm_amd_padded_row_size_in_bytes(Ds[t % 4], tys[t % 4], 16, 4);
    off += (row * 100 + 127) / 128 * 128;
  }
  p.bytes = off;
  return p;
}

struct Buffers {
  void *weights, *indices, *offsets, *out, *status;
  Buffers(const Problem& p, int64_t B, int64_t n) {
    CHECK(hipMalloc(&weights, p.bytes) == hipSuccess);
    CHECK(hipMalloc(&indices, 8 * (n + 1)) == hipSuccess);
    CHECK(hipMalloc(&offsets, 8 * (p.T * B + 1)) == hipSuccess);
    CHECK(hipMalloc(&out, 4 * B * (p.D_offsets.back() + 8 * p.T)) == hipSuccess);
    CHECK(hipMalloc(&status, 16) == hipSuccess);
  }
  ~Buffers() {
    hipFree(weights);
    hipFree(indices);
    hipFree(offsets);
    hipFree(out);
    hipFree(status);
  }
};

int forward(fbgemm_amd_tbe_plan* plan, const Problem& p, Buffers& b, int64_t B, int64_t n, hipStream_t s, int32_t out_ty = 1) {
  return fbgemm_amd_tbe_forward(plan, b.weights, nullptr, b.indices, b.offsets, 64, n, p.T * B + 1, 0, nullptr, out_ty, b.out, b.status, s);
}

void plan_create_failures() {
  const Problem p = make_problem(5);
  fbgemm_amd_tbe_plan* plan = nullptr;
  CHECK(fbgemm_amd_tbe_plan_create(&plan, 0, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) < 0);
  CHECK(fbgemm_amd_tbe_plan_create(nullptr, 5, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) < 0);
  std::vector<uint8_t> bad_ty = p.tys;
  bad_ty[3] = 42; // rejected after the tables before it were filled in
  CHECK(fbgemm_amd_tbe_plan_create(&plan, 5, p.wo.data(), bad_ty.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) < 0);
  std::vector<int32_t> bad_D = p.D_offsets;
  bad_D[4] = bad_D[3];
  CHECK(fbgemm_amd_tbe_plan_create(&plan, 5, p.wo.data(), p.tys.data(), bad_D.data(), nullptr, p.bytes, 0, 16) < 0);
  // every allocation of a creation fails in turn: what was made before it goes back
  for (long k = 0; k < 8; ++k) {
    hip_stub_fail_malloc_after(k);
    plan = nullptr;
    const int rc = fbgemm_amd_tbe_plan_create(&plan, 5, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16);
    hip_stub_fail_malloc_after(-1);
    if (rc == 0) fbgemm_amd_tbe_plan_destroy(plan);
    else CHECK(plan == nullptr);
    CHECK(hip_stub_live_allocations() == 0);
  }
  fbgemm_amd_tbe_plan_destroy(nullptr);
}

void work_list_cache_and_graphs() {
  const Problem p = make_problem(6);
  fbgemm_amd_tbe_plan* plan = nullptr;
  CHECK(fbgemm_amd_tbe_plan_create(&plan, p.T, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) == 0);
  const int64_t big_n = 1 << 21; // from here on the forwards order their bags (per-stream scratch)
  Buffers b(p, 64, big_n);
  hipStream_t s0 = hip_stub_stream(0), s1 = hip_stub_stream(1), s2 = hip_stub_stream(2);
  // a new batch size under capture is refused (it would allocate); nothing is left behind
  hip_stub_set_capturing(s0, true);
  CHECK(forward(plan, p, b, 7, big_n, s0) < 0);
  hip_stub_set_capturing(s0, false);
  CHECK(fbgemm_amd_tbe_plan_cached_work(plan) == 0);
  // batch sizes 1..6 on three streams, then some of them under capture (pinned)
  for (int64_t B = 1; B <= 6; ++B)
    for (hipStream_t s : {s0, s1, s2}) CHECK(forward(plan, p, b, B, big_n, s) == 0);
  hip_stub_set_capturing(s1, true);
  for (int64_t B : {2, 4}) CHECK(forward(plan, p, b, B, big_n, s1) == 0);
  hip_stub_set_capturing(s1, false);
  CHECK(fbgemm_amd_tbe_plan_pinned_work(plan) == 2);
  // many more batch sizes: the cache stays bounded, the pinned entries stay, the forwards go on working
  for (int64_t B = 7; B <= 48; ++B) CHECK(forward(plan, p, b, B, big_n, B % 2 ? s0 : s2) == 0);
  CHECK(fbgemm_amd_tbe_plan_cached_work(plan) <= 16);
  CHECK(fbgemm_amd_tbe_plan_pinned_work(plan) == 2);
  hip_stub_set_capturing(s1, true);
  CHECK(forward(plan, p, b, 2, big_n, s1) == 0); // a replayed graph's entry is still there
  hip_stub_set_capturing(s1, false);
  // small forwards (no scheduler), the three lane-shape variants, the 8-bit pooled output
  CHECK(forward(plan, p, b, 3, 100, s0) == 0);
  CHECK(fbgemm_amd_set_narrow_below_waves(0) == 0);
  CHECK(forward(plan, p, b, 3, 100, s0) == 0);
  CHECK(fbgemm_amd_set_narrow_below_waves(-1) == 0);
  CHECK(fbgemm_amd_set_lean(0) == 0);
  CHECK(forward(plan, p, b, 3, big_n, s0) == 0);
  CHECK(fbgemm_amd_set_lean(-1) == 0);
  CHECK(forward(plan, p, b, 5, big_n, s0, /*INT8 output*/ 2) == 0);
  CHECK(forward(plan, p, b, 40, big_n, s0, 2) == 0); // the scratch of the 8-bit output grows
  CHECK(forward(plan, p, b, 40, big_n, s1, 2) == 0); // another stream: waits for the event behind the last use
  hip_stub_set_capturing(s2, true);
  CHECK(forward(plan, p, b, 40, big_n, s2, 2) == 0); // under capture nothing is recorded or waited for
  hip_stub_set_capturing(s2, false);
  CHECK(fbgemm_amd_tbe_plan_reuse_order(plan, 1) == 0);
  CHECK(forward(plan, p, b, 5, big_n, s0) == 0);
  CHECK(fbgemm_amd_tbe_plan_reuse_order(plan, 0) == 0);
  // trim drops everything, also what graphs hold; the plan works afterwards
  CHECK(fbgemm_amd_tbe_plan_trim(plan) == 0);
  CHECK(fbgemm_amd_tbe_plan_cached_work(plan) == 0);
  CHECK(forward(plan, p, b, 2, big_n, s1) == 0);
  fbgemm_amd_tbe_plan_destroy(plan);
}

void remappings_twice_and_split_bags() {
  Problem p = make_problem(4);
  for (auto& ty : p.tys) ty = 3; // 4-bit tables only: the tolerance-grade plan cuts long bags into segments
  p.D_offsets = {0, 64, 192, 448, 512};
  p.wo = {0, 8192, 32768, 65536};
  p.bytes = 131072;
  fbgemm_amd_tbe_plan* plan = nullptr;
  CHECK(fbgemm_amd_tbe_plan_create(&plan, p.T, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) == 0);
  CHECK(fbgemm_amd_tbe_plan_set_accumulate(plan, FBGEMM_AMD_ACC_FAST) == 0);
  Buffers b(p, 8, 4096);
  hipStream_t s = hip_stub_stream(3);
  const std::vector<int64_t> remap_off = {0, 1000, 1000, 3000, 3500}; // table 1 is not pruned
  void* remap = nullptr;
  CHECK(hipMalloc(&remap, 4 * 3500) == hipSuccess);
  void* d_remap_off = nullptr;
  CHECK(hipMalloc(&d_remap_off, 8 * 5) == hipSuccess);
  hipMemcpy(d_remap_off, remap_off.data(), 8 * 5, hipMemcpyHostToDevice);
  auto pruned = [&](int64_t B, int64_t n) {
    return fbgemm_amd_tbe_forward_pruned(plan, b.weights, nullptr, b.indices, b.offsets, 64, n, p.T * B + 1, 1, nullptr, 0, b.out,
                                         remap, 32, (const int64_t*)d_remap_off, 5, b.status, s);
  };
  CHECK(pruned(2, 4096) == 0); // few long bags: split into segments (plan-owned scratch), mappings read as arrays
  CHECK(fbgemm_amd_tbe_plan_set_index_remappings(plan, remap, 32, remap_off.data(), 5, s) == 0);
  CHECK(fbgemm_amd_tbe_plan_rank_tables(plan) == 3);
  CHECK(pruned(2, 4096) == 0);
  CHECK(fbgemm_amd_tbe_plan_set_index_remappings(plan, remap, 32, remap_off.data(), 5, s) == 0); // the records are made again
  CHECK(pruned(2, 4096) == 0);
  CHECK(pruned(8, 4096) == 0); // more bags: the segment scratch grows
  CHECK(fbgemm_amd_tbe_plan_set_index_remappings(plan, nullptr, 32, nullptr, 0, s) == 0);  // and dropped
  CHECK(fbgemm_amd_tbe_plan_rank_tables(plan) == 0);
  CHECK(pruned(2, 4096) == 0);
  CHECK(fbgemm_amd_tbe_plan_set_index_remappings(plan, remap, 32, remap_off.data(), 4, s) < 0); // wrong number of offsets
  fbgemm_amd_tbe_plan_destroy(plan);
  hipFree(remap);
  hipFree(d_remap_off);
}

fbgemm_amd_spmdm_config single_table(int32_t ty, int64_t D, int32_t use_offsets, int32_t accumulate) {
  fbgemm_amd_spmdm_config c;
  memset(&c, 0, sizeof(c));
  c.weight_ty = ty;
  c.output_ty = 0;
  c.index_bits = 64;
  c.offset_bits = 32;
  c.block_size = D;
  c.output_stride = -1;
  c.input_stride = -1;
  c.use_offsets = use_offsets;
  c.scale_bias_last = 1;
  c.accumulate = accumulate;
  return c;
}

void one_thread_of_single_table_calls(int id) {
  void *table, *idx, *lens, *out;
  CHECK(hipMalloc(&table, 1 << 20) == hipSuccess);
  CHECK(hipMalloc(&idx, 8 << 22) == hipSuccess);
  CHECK(hipMalloc(&lens, 4 * 70001) == hipSuccess);
  CHECK(hipMalloc(&out, 4 * 70000 * 128) == hipSuccess);
  hipStream_t s = hip_stub_stream(4 + id);
  // lengths instead of offsets (the prefix sum lives in the thread's scratch, which grows), a call
  // large enough to order its bags, few long bags in the tolerance-grade mode (segments)
  for (int64_t bags : {10, 3000, 70000}) {
    fbgemm_amd_spmdm_config c = single_table(3, 128, 0, FBGEMM_AMD_ACC_EXACT);
    CHECK(fbgemm_amd_spmdm_run(&c, bags, 1 << 22, 1000, table, idx, lens, nullptr, out, nullptr, s) >= 0);
  }
  fbgemm_amd_spmdm_config c = single_table(3, 128, 1, FBGEMM_AMD_ACC_FAST);
  CHECK(fbgemm_amd_spmdm_run(&c, 4, 4000, 1000, table, idx, lens, nullptr, out, nullptr, s) >= 0);
  CHECK(fbgemm_amd_spmdm_run(&c, 40, 40000, 1000, table, idx, lens, nullptr, out, nullptr, s) >= 0);
  hipFree(table);
  hipFree(idx);
  hipFree(lens);
  hipFree(out);
}

void thread_scratch_hand_over() {
  for (int round = 0; round < 3; ++round) { // threads that end hand their scratch to the next ones
    std::vector<std::thread> ts;
    for (int i = 0; i < 3; ++i) ts.emplace_back(one_thread_of_single_table_calls, i);
    for (auto& t : ts) t.join();
  }
  one_thread_of_single_table_calls(7); // and this thread adopts a set too
}

void entry_point_that_allocates_nothing() {
  void *table, *idx, *lens, *out, *status;
  CHECK(hipMalloc(&table, 1 << 20) == hipSuccess);
  CHECK(hipMalloc(&idx, 8 << 22) == hipSuccess);
  CHECK(hipMalloc(&lens, 4 * 65537) == hipSuccess);
  CHECK(hipMalloc(&out, 4 * 65536 * 128) == hipSuccess);
  CHECK(hipMalloc(&status, 16) == hipSuccess);
  const long before = hip_stub_total_allocations();
  fbgemm_amd_spmdm_config c = single_table(3, 128, 0, FBGEMM_AMD_ACC_EXACT);
  const int64_t most = fbgemm_amd_noalloc_max_bags();
  CHECK(fbgemm_amd_spmdm_launch_noalloc(&c, most, 1 << 22, 1000, table, idx, lens, nullptr, out, nullptr, status, nullptr) == 0);
  CHECK(fbgemm_amd_spmdm_launch_noalloc(&c, 100, 1 << 22, 1000, table, idx, lens, nullptr, out, nullptr, status, nullptr) == 0);
  CHECK(fbgemm_amd_spmdm_launch_noalloc(&c, most + 1, 1 << 22, 1000, table, idx, lens, nullptr, out, nullptr, status, nullptr) < 0);
  CHECK(hip_stub_total_allocations() == before); // it allocated nothing
  hipFree(table);
  hipFree(idx);
  hipFree(lens);
  hipFree(out);
  hipFree(status);
}

void allocation_failures_in_a_first_forward() {
  const Problem p = make_problem(5);
  Buffers b(p, 16, 1 << 21);
  hipStream_t s = hip_stub_stream(9);
  const long base = hip_stub_live_allocations();
  for (long k = 0; k < 24; ++k) {
    fbgemm_amd_tbe_plan* plan = nullptr;
    CHECK(fbgemm_amd_tbe_plan_create(&plan, p.T, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) == 0);
    hip_stub_fail_malloc_after(k);
    const int rc = forward(plan, p, b, 16, 1 << 21, s);
    const int rc8 = forward(plan, p, b, 16, 1 << 21, s, 2);
    hip_stub_fail_malloc_after(-1);
    (void)rc;
    (void)rc8;
    CHECK(forward(plan, p, b, 16, 1 << 21, s) == 0); // a plan whose forward failed half-way works once memory is there
    fbgemm_amd_tbe_plan_destroy(plan);
    CHECK(hip_stub_live_allocations() == base);
  }
}

// A plan whose tables all have 4-bit rows in bags of 8 lanes: forwards that order their bags take the
// lean kernel's four-waves-per-SIMD instance, whose redo queue is made with every bag-order buffer
// (three streams, allocation failures in between) and freed with the work set.
void plan_of_wide_4bit_tables() {
  Problem p;
  p.T = 3;
  int64_t off = 0;
  p.D_offsets.push_back(0);
  for (int t = 0; t < p.T; ++t) {
    p.wo.push_back(off);
    p.tys.push_back(3);
    p.D_offsets.push_back(p.D_offsets.back() + 256);
    off += (fbgemm_amd_padded_row_size_in_bytes(256, 3, 16, 4) * 100 + 127) / 128 * 128;
  }
  p.bytes = off;
  // about 19 rows per bag: enough lookups for the bag order, bags too short for the end-to-end lane shapes
  const int64_t big_n = 1 << 21, B = 36000;
  Buffers b(p, B, big_n);
  const long base = hip_stub_live_allocations();
  CHECK(fbgemm_amd_set_wide4(2) == 0); // always that instance
  for (long k = -1; k < 12; ++k) {
    fbgemm_amd_tbe_plan* plan = nullptr;
    CHECK(fbgemm_amd_tbe_plan_create(&plan, p.T, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) == 0);
    hip_stub_fail_malloc_after(k);
    (void)forward(plan, p, b, B, big_n, hip_stub_stream(0));
    hip_stub_fail_malloc_after(-1);
    for (int s = 0; s < 3; ++s) CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(s)) == 0);
    CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(1), /*INT8 output*/ 2) == 0);
    CHECK(forward(plan, p, b, 48, 100, hip_stub_stream(1)) == 0); // a small forward: no bag order, no queue
    fbgemm_amd_tbe_plan_destroy(plan);
    CHECK(hip_stub_live_allocations() == base);
  }
  CHECK(hip_stub_wide4_launches() >= 13 * 3); // the forwards above did take that instance
  // The default: the first forwards of a batch size time the two kernels in turn (waiting for the second event),
  // then the faster one stays. Under capture nothing is measured.
  CHECK(fbgemm_amd_set_wide4(-1) == 0);
  for (int faster = 0; faster < 2; ++faster) {
    hip_stub_set_elapsed_ms(1.0f, faster ? 0.5f : 0.995f); // the four-wave instance has to win by 1 %
    fbgemm_amd_tbe_plan* plan = nullptr;
    CHECK(fbgemm_amd_tbe_plan_create(&plan, p.T, p.wo.data(), p.tys.data(), p.D_offsets.data(), nullptr, p.bytes, 0, 16) == 0);
    CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(0)) == 0);
    hip_stub_set_capturing(hip_stub_stream(1), true);
    const long before_capture = hip_stub_wide4_launches();
    CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(1)) == 0); // undecided and capturing: the general-purpose kernel
    CHECK(hip_stub_wide4_launches() == before_capture);
    hip_stub_set_capturing(hip_stub_stream(1), false);
    for (int i = 0; i < 24; ++i) CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(i % 3)) == 0);
    const long settled = hip_stub_wide4_launches();
    for (int i = 0; i < 6; ++i) CHECK(forward(plan, p, b, B, big_n, hip_stub_stream(i % 3)) == 0);
    CHECK(hip_stub_wide4_launches() - settled == (faster ? 6 : 0));
    fbgemm_amd_tbe_plan_destroy(plan);
    CHECK(hip_stub_live_allocations() == base);
  }
}

} // namespace

int main() {
  plan_of_wide_4bit_tables();
  plan_create_failures();
  work_list_cache_and_graphs();
  remappings_twice_and_split_bags();
  thread_scratch_hand_over();
  entry_point_that_allocates_nothing();
  allocation_failures_in_a_first_forward();
  printf("launches %ld, device allocations %ld\n", hip_stub_launches(), hip_stub_total_allocations());
  printf("PASSED\n");
  return 0;
}
