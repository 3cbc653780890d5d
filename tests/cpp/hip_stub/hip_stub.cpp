// Definitions behind tests/cpp/hip_stub/hip/hip_runtime.h, and stand-ins for the
// kernel launchers of fbgemm_amd/csrc/launchers.h: they launch nothing and leave in
// "device" memory only what the host code reads back afterwards.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>

#include "../../../fbgemm_amd/csrc/launchers.h"

namespace {
std::mutex g_mu;
std::set<void*> g_live;
std::set<hipStream_t> g_capturing;
std::atomic<long> g_total{0}, g_launches{0}, g_fail_after{-1}, g_wide4{0};
std::atomic<int> g_last_lean_wide4{0};
std::atomic<float> g_elapsed_general{1.0f}, g_elapsed_wide4{1.0f};
struct Obj { int kind; };
} // namespace

struct hipStubStream { int id; };
struct hipStubEvent { int id; };

hipError_t hipMalloc(void** p, size_t bytes) {
  long f = g_fail_after.load();
  if (f >= 0) {
    g_fail_after.store(f - 1);
    if (f == 0) {
      *p = nullptr;
      return hipErrorOutOfMemory;
    }
  }
  *p = malloc(bytes ? bytes : 1);
  if (!*p) return hipErrorOutOfMemory;
  memset(*p, 0xa5, bytes); // what a kernel has not written yet
  std::lock_guard<std::mutex> lk(g_mu);
  g_live.insert(*p);
  ++g_total;
  return hipSuccess;
}
hipError_t hipFree(void* p) {
  if (!p) return hipSuccess;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    g_live.erase(p); // a pointer that is not there is the sanitizer's to report, in free()
  }
  free(p);
  return hipSuccess;
}
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind) {
  if (bytes) memcpy(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind, hipStream_t) {
  if (bytes) memcpy(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t) {
  if (bytes) memset(dst, value, bytes);
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }
hipError_t hipGetDevice(int* dev) {
  *dev = 0;
  return hipSuccess;
}
hipError_t hipGetLastError(void) { return hipSuccess; }
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : e == hipErrorOutOfMemory ? "out of memory" : "error"; }
hipError_t hipStreamIsCapturing(hipStream_t stream, hipStreamCaptureStatus* status) {
  std::lock_guard<std::mutex> lk(g_mu);
  *status = g_capturing.count(stream) ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
  return hipSuccess;
}
hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned) {
  *stream = new hipStubStream{-1};
  return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
  delete stream;
  return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t event, unsigned) { return event ? hipSuccess : hipErrorInvalidValue; }
hipError_t hipEventCreateWithFlags(hipEvent_t* event, unsigned) {
  *event = new hipStubEvent{0};
  return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t event) {
  delete event;
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t event, hipStream_t) {
  event->id++; // touches the event: a destroyed one is the sanitizer's to report
  return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t event) {
  if (!event) return hipErrorInvalidValue;
  (void)event->id;
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t start, hipEvent_t stop) {
  if (!start || !stop) return hipErrorInvalidValue;
  (void)start->id;
  (void)stop->id;
  *ms = g_last_lean_wide4.load() ? g_elapsed_wide4.load() : g_elapsed_general.load();
  return hipSuccess;
}
hipError_t hipGetSymbolAddressStub(void** p, const void* symbol) {
  *p = const_cast<void*>(symbol);
  return hipSuccess;
}

void hip_stub_set_capturing(hipStream_t stream, bool on) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (on) g_capturing.insert(stream);
  else g_capturing.erase(stream);
}
void hip_stub_fail_malloc_after(long n) { g_fail_after.store(n); }
long hip_stub_live_allocations(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  return (long)g_live.size();
}
long hip_stub_total_allocations(void) { return g_total.load(); }
long hip_stub_launches(void) { return g_launches.load(); }
long hip_stub_wide4_launches(void) { return g_wide4.load(); }
void hip_stub_set_elapsed_ms(float general_ms, float wide4_ms) {
  g_elapsed_general = general_ms;
  g_elapsed_wide4 = wide4_ms;
}
hipStream_t hip_stub_stream(int id) {
  static hipStubStream streams[16];
  return &streams[id & 15];
}

// ---- launchers: nothing runs; the words the host reads back are written ---------------------
namespace fbgemm_amd {
#define LAUNCHED() (++g_launches, hipSuccess)
hipError_t launch_lookup(const LookupArgs& a, bool, hipStream_t) {
  // what a kernel would dereference must still be alive: touch the first bytes of each list
  if (a.work) (void)*(volatile const int32_t*)&a.work[0].table;
  if (a.xcd_start) (void)*(volatile const int64_t*)&a.xcd_start[8];
  if (a.order) (void)*(volatile const int64_t*)&a.order[0].o0;
  if (a.tables) (void)*(volatile const int64_t*)&a.tables[0].row_stride;
  if (a.rank_records) (void)*(volatile const uint32_t*)&a.rank_records[0].bits;
  if (a.rank_offsets) (void)*(volatile const int64_t*)&a.rank_offsets[0];
  return LAUNCHED();
}
hipError_t launch_lookup_lean(const LookupArgs& a, bool idx64, bool, bool wide4, hipStream_t s) {
  if (wide4) { // the redo queue of that instance must be there, and as long as the work list
    if (!a.redo || !a.redo_count) return hipErrorInvalidValue;
    (void)*(volatile const int32_t*)&a.redo_count[1];
    (void)*(volatile const int32_t*)&a.redo[a.num_waves - 1].first_bag;
    ++g_wide4;
  }
  g_last_lean_wide4 = wide4 ? 1 : 0;
  return launch_lookup(a, idx64, s);
}
hipError_t launch_lengths_to_offsets(const void*, bool, int64_t n, int64_t* offsets, hipStream_t) {
  for (int64_t i = 0; i <= n; ++i) offsets[i] = 0; // the whole buffer must be there
  return LAUNCHED();
}
hipError_t launch_status_clear(Status* st, hipStream_t) {
  st->bits = 0;
  st->pad = 0;
  st->first_bad_pos = ~0ull;
  return LAUNCHED();
}
hipError_t launch_bag_order(const void*, bool, int32_t B, int32_t T, BagEntry* order, hipStream_t) {
  memset(order, 0, sizeof(BagEntry) * (size_t)B * (size_t)T);
  return LAUNCHED();
}
hipError_t launch_sequence_lookup(const TableDesc*, const uint8_t*, const uint8_t*, const void*, bool, const void*, int32_t, int32_t,
                                  int64_t, int32_t, int32_t, void*, int32_t, float, Status*, hipStream_t) { return LAUNCHED(); }
hipError_t launch_row_lookup(const TableDesc&, const uint8_t*, const void*, bool, const float*, int64_t, int32_t, void*, int64_t,
                             int64_t, int32_t, float, Status*, hipStream_t) { return LAUNCHED(); }
hipError_t launch_float_to_hfp8(const float*, int64_t, int32_t, int32_t, float, uint8_t*, hipStream_t) { return LAUNCHED(); }
hipError_t launch_hfp8_to_float(const uint8_t*, int64_t, int32_t, int32_t, float*, hipStream_t) { return LAUNCHED(); }
hipError_t launch_inplace_update(const TableDesc*, int32_t, uint8_t*, uint8_t*, const uint8_t*, int64_t, const int32_t*, const void*,
                                 bool, const int64_t*, int64_t, int64_t, Status*, hipStream_t) { return LAUNCHED(); }
hipError_t launch_remap_row_idx(const void*, bool, const int32_t*, const void*, bool, const int64_t*, int32_t, int64_t, void*,
                                hipStream_t) { return LAUNCHED(); }
int64_t prune_partials(int64_t rows) { return rows / 1024 + 2; }
hipError_t launch_split_offsets(const void*, bool, int64_t bags, int32_t K, bool, int64_t, int64_t* voff, Status*, hipStream_t) {
  for (int64_t i = 0; i <= bags * K; ++i) voff[i] = 0;
  return LAUNCHED();
}
hipError_t launch_combine_segments(const float* partial, int64_t partial_stride, int32_t B, int32_t K, int32_t, const int32_t*, int32_t,
                                   const void*, bool, bool, void*, int32_t, int64_t, hipStream_t) {
  (void)*(volatile const float*)&partial[(int64_t)B * K * partial_stride - 1];
  return LAUNCHED();
}
int64_t remap_rank_words(int64_t rows) { return (rows + 31) / 32; }
int64_t remap_rank_partials(int64_t rows) { return rows / 2048 + 2; }
hipError_t launch_remap_rank_build(const void*, bool, int64_t rows, RankRecord* records, int64_t* partial, int32_t* not_monotone,
                                   hipStream_t) {
  memset(records, 0, sizeof(RankRecord) * (size_t)remap_rank_words(rows));
  partial[remap_rank_partials(rows) - 1] = 0;
  *not_monotone = 0; // an order-preserving mapping: the records are used
  return LAUNCHED();
}
hipError_t launch_prune_map(const float*, int64_t, double, int, int64_t, bool, void*, int64_t* num_kept, int64_t*, hipStream_t) {
  *num_kept = 0;
  return LAUNCHED();
}
hipError_t launch_prune_gather(const void*, int64_t, int64_t, const void*, bool, void*, int64_t, hipStream_t) { return LAUNCHED(); }
hipError_t launch_compressed_indices_remap(const void*, bool, const int32_t*, int64_t, const void*, int64_t, const float*, int64_t,
                                           int64_t, void*, void*, float*, int64_t* before, int64_t*, int32_t*, Status*, hipStream_t) {
  if (before) before[0] = 0;
  return LAUNCHED();
}
hipError_t launch_quantize_segments(const float* input, int64_t lines, int32_t, const int32_t*, int32_t total_D, int32_t, uint8_t*,
                                    const int32_t*, int32_t, hipStream_t) {
  (void)*(volatile const float*)&input[lines * total_D - 1];
  return LAUNCHED();
}
hipError_t launch_bounds_check(const int64_t*, int32_t, void*, void*, bool, int64_t, int64_t, int64_t, const int32_t*, int, int64_t*,
                               int64_t*, int64_t*, Status*, hipStream_t) { return LAUNCHED(); }
int64_t bounds_check_partials(int64_t total_B) { return total_B / 1024 + 2; }
hipError_t launch_quantize_rowwise(const void*, bool, int64_t, int32_t, int32_t, int32_t, int32_t, int64_t, void*, const void*,
                                   hipStream_t) { return LAUNCHED(); }
hipError_t launch_dequantize_rowwise(const void*, int64_t, int64_t, int32_t, int32_t, int32_t, int32_t, int32_t, void*, hipStream_t) {
  return LAUNCHED();
}
hipError_t launch_pruned_hashmap_lookup(const void*, const void*, bool, const void*, bool, const int64_t*, int32_t, int32_t, void*,
                                        hipStream_t) { return LAUNCHED(); }
hipError_t launch_pruned_array_lookup(const void*, const void*, bool, const void*, bool, const int64_t*, int32_t, int32_t, void*,
                                      hipStream_t) { return LAUNCHED(); }
} // namespace fbgemm_amd
