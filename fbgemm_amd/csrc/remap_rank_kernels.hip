// A compact form of the pruned-row mapping for the fused remap of the
// table-batched forward. No counterpart in the reference, which keeps one int32
// per logical row (index_remappings_array, the argument of pruned_array_lookup):
// a lookup then pays a 128-byte line from a table-sized array for 4 bytes.
//
// Where a table's mapping is ORDER-PRESERVING (the kept rows are numbered 0, 1,
// 2, ... in logical order; what embedding_bag_rowwise_prune, the inference
// converter and the reference's test generator all produce), the physical row
// is the number of kept rows in front of the logical one. That rank is stored as
// one 8-byte record per 32 logical rows: {kept rows before the record's first
// row, a bit per row}, 2 bits per logical row instead of 32, small enough to
// stay in the L2 of the XCD that owns the table:
//     kept     = (bits >> (id & 31)) & 1
//     physical = before + popcount(bits & ((1 << (id & 31)) - 1))
// The records are built on the device from the int32 / int64 mapping in three
// launches (per-word bits and counts, a scan of the workgroup totals, the
// records) and every kept row's mapping entry is compared with its rank: one
// mismatch marks the table as not order-preserving and the forward keeps reading
// its array. Integer arithmetic throughout: results are identical to the array's.
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

constexpr int RR_THREADS = 256; // one 32-row word per thread

template <typename remap_t>
__device__ __forceinline__ uint32_t word_bits(const remap_t* mapping, int64_t rows, int64_t w) {
  uint32_t bits = 0;
  const int64_t r0 = w * 32;
  for (int b = 0; b < 32; ++b) {
    const int64_t r = r0 + b;
    if (r < rows && mapping[r] != (remap_t)-1) bits |= 1u << b;
  }
  return bits;
}

__device__ __forceinline__ uint32_t block_inclusive_sum_u32(uint32_t mine, uint32_t* lds) {
  lds[threadIdx.x] = mine;
  __syncthreads();
  for (int step = 1; step < RR_THREADS; step <<= 1) {
    const uint32_t o = (int)threadIdx.x >= step ? lds[threadIdx.x - step] : 0u;
    __syncthreads();
    lds[threadIdx.x] += o;
    __syncthreads();
  }
  return lds[threadIdx.x];
}

// pass 1: the bits of every word, the kept rows of every workgroup's words
template <typename remap_t>
__global__ __launch_bounds__(RR_THREADS) void remap_rank_count_kernel(const remap_t* mapping, int64_t rows, int64_t words,
                                                                      RankRecord* records, int64_t* partial) {
  __shared__ uint32_t lds[RR_THREADS];
  const int64_t w = (int64_t)blockIdx.x * RR_THREADS + threadIdx.x;
  uint32_t bits = 0;
  if (w < words) {
    bits = word_bits(mapping, rows, w);
    records[w].bits = bits;
  }
  const uint32_t incl = block_inclusive_sum_u32((uint32_t)__builtin_popcount(bits), lds);
  if (threadIdx.x == RR_THREADS - 1) partial[blockIdx.x] = incl;
}

// pass 2: exclusive prefix sum of the workgroup totals, one workgroup
__global__ __launch_bounds__(1024) void remap_rank_scan_kernel(int64_t* partial, int64_t n) {
  __shared__ int64_t lds[1024];
  const int tid = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = (int64_t)tid * per, hi = lo + per < n ? lo + per : n;
  int64_t sum = 0;
  for (int64_t i = lo; i < hi; ++i) sum += partial[i];
  lds[tid] = sum;
  __syncthreads();
  for (int step = 1; step < 1024; step <<= 1) {
    const int64_t o = tid >= step ? lds[tid - step] : 0;
    __syncthreads();
    lds[tid] += o;
    __syncthreads();
  }
  int64_t run = lds[tid] - sum;
  for (int64_t i = lo; i < hi; ++i) {
    const int64_t v = partial[i];
    partial[i] = run;
    run += v;
  }
}

// pass 3: the records, and the check that the mapping IS the rank
template <typename remap_t>
__global__ __launch_bounds__(RR_THREADS) void remap_rank_build_kernel(const remap_t* mapping, int64_t rows, int64_t words,
                                                                      RankRecord* records, const int64_t* partial,
                                                                      int32_t* not_monotone) {
  __shared__ uint32_t lds[RR_THREADS];
  const int64_t w = (int64_t)blockIdx.x * RR_THREADS + threadIdx.x;
  const uint32_t bits = w < words ? records[w].bits : 0u;
  const uint32_t cnt = (uint32_t)__builtin_popcount(bits);
  const uint32_t incl = block_inclusive_sum_u32(cnt, lds);
  if (w >= words) return;
  const int64_t before = partial[blockIdx.x] + (int64_t)(incl - cnt);
  bool bad = before > 0x7fffffffLL;
  records[w].before = (uint32_t)before;
  const int64_t r0 = w * 32;
  for (int b = 0; b < 32; ++b) {
    if ((bits >> b) & 1u) {
      const int64_t want = before + __builtin_popcount(bits & ((1u << b) - 1u));
      bad = bad || (int64_t)mapping[r0 + b] != want;
    }
  }
  if (bad) atomicOr(not_monotone, 1);
}

} // namespace

int64_t remap_rank_words(int64_t rows) { return (rows + 31) / 32; }
int64_t remap_rank_partials(int64_t rows) { return (remap_rank_words(rows) + RR_THREADS - 1) / RR_THREADS; }

// Records of one table: `records` holds remap_rank_words(rows) entries, `partial`
// remap_rank_partials(rows) scratch entries, *not_monotone is ORed with 1 when the
// mapping is not order-preserving.
hipError_t launch_remap_rank_build(const void* mapping, bool remap64, int64_t rows, RankRecord* records, int64_t* partial,
                                   int32_t* not_monotone, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  const int64_t words = remap_rank_words(rows);
  const int64_t blocks = remap_rank_partials(rows);
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  if (remap64)
    hipLaunchKernelGGL(remap_rank_count_kernel<int64_t>, dim3((unsigned)blocks), dim3(RR_THREADS), 0, stream,
                       (const int64_t*)mapping, rows, words, records, partial);
  else
    hipLaunchKernelGGL(remap_rank_count_kernel<int32_t>, dim3((unsigned)blocks), dim3(RR_THREADS), 0, stream,
                       (const int32_t*)mapping, rows, words, records, partial);
  hipLaunchKernelGGL(remap_rank_scan_kernel, dim3(1), dim3(1024), 0, stream, partial, blocks);
  if (remap64)
    hipLaunchKernelGGL(remap_rank_build_kernel<int64_t>, dim3((unsigned)blocks), dim3(RR_THREADS), 0, stream,
                       (const int64_t*)mapping, rows, words, records, partial, not_monotone);
  else
    hipLaunchKernelGGL(remap_rank_build_kernel<int32_t>, dim3((unsigned)blocks), dim3(RR_THREADS), 0, stream,
                       (const int32_t*)mapping, rows, words, records, partial, not_monotone);
  return hipGetLastError();
}

} // namespace fbgemm_amd
