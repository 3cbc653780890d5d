// gfx950 kernels of the index operators that run before the lookup:
// bounds_check_indices and pruned_hashmap_lookup.
//
// bounds_check_indices follows the reference's CPU operator
// (fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:76-219), whose
// loop over the bags is sequential: repairing a bag writes both of its offsets,
// and the next bag starts from the repaired value. Carried through, the offsets
// it leaves are the running maximum of the original offsets clamped to
// [0, num_indices] (the last one replaced by num_indices first), and a bag is
// "bad" (one warning) when the running maximum at its start exceeds its
// original end, or that end exceeds num_indices, or the very first offset is
// negative. A running maximum is a scan, so the GPU computes exactly what the
// sequential loop does, independent of scheduling. (The reference's own GPU
// kernel lets neighbouring bags race on the shared offset.)
#include <hip/hip_runtime.h>

#include <type_traits>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

constexpr int SCAN_THREADS = 1024;
constexpr int SCAN_ITEMS = 4; // offsets per thread
constexpr int SCAN_BLOCK = SCAN_THREADS * SCAN_ITEMS;

__device__ __forceinline__ int64_t read_index(const void* p, bool is64, int64_t i) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}
__device__ __forceinline__ void write_index(void* p, bool is64, int64_t i, int64_t v) {
  if (is64) reinterpret_cast<int64_t*>(p)[i] = v;
  else reinterpret_cast<int32_t*>(p)[i] = (int32_t)v;
}

// offsets[k] as the scan sees it: the last one is num_indices, all are clamped
__device__ __forceinline__ int64_t clamped_offset(const void* offsets, bool is64, int64_t k, int64_t total_B, int64_t N) {
  int64_t v = k == total_B ? N : read_index(offsets, is64, k);
  v = v < N ? v : N;
  return v > 0 ? v : 0;
}

__device__ __forceinline__ int64_t block_max(int64_t v, int64_t* lds) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int step = SCAN_THREADS / 2; step > 0; step >>= 1) {
    if (tid < step) lds[tid] = lds[tid] > lds[tid + step] ? lds[tid] : lds[tid + step];
    __syncthreads();
  }
  const int64_t r = lds[0];
  __syncthreads();
  return r;
}

// pass 1: maximum of the clamped offsets of every block of SCAN_BLOCK offsets
__global__ __launch_bounds__(SCAN_THREADS) void bounds_partial_max_kernel(
    const void* offsets, int is64, int64_t total_B, int64_t N, int64_t* partial, int64_t* warning, int mode) {
  __shared__ int64_t lds[SCAN_THREADS];
  if (mode == 1 && blockIdx.x == 0 && threadIdx.x == 0) warning[0] = 0; // WARNING mode starts from zero
  const int64_t base = (int64_t)blockIdx.x * SCAN_BLOCK + (int64_t)threadIdx.x * SCAN_ITEMS;
  int64_t m = 0;
  for (int i = 0; i < SCAN_ITEMS; ++i) {
    const int64_t k = base + i;
    if (k <= total_B) {
      const int64_t v = clamped_offset(offsets, is64, k, total_B, N);
      m = v > m ? v : m;
    }
  }
  m = block_max(m, lds);
  if (threadIdx.x == 0) partial[blockIdx.x] = m;
}

// pass 2 (one workgroup): partial[b] becomes the maximum of all blocks before b
__global__ __launch_bounds__(SCAN_THREADS) void bounds_carry_kernel(int64_t* partial, int64_t nblocks) {
  __shared__ int64_t lds[SCAN_THREADS];
  int64_t carry = 0;
  for (int64_t b0 = 0; b0 < nblocks; b0 += SCAN_THREADS) {
    const int64_t b = b0 + threadIdx.x;
    const int64_t mine = b < nblocks ? partial[b] : 0;
    lds[threadIdx.x] = mine;
    __syncthreads();
    for (int step = 1; step < SCAN_THREADS; step <<= 1) {
      const int64_t v = (int)threadIdx.x >= step ? lds[threadIdx.x - step] : 0;
      __syncthreads();
      lds[threadIdx.x] = lds[threadIdx.x] > v ? lds[threadIdx.x] : v;
      __syncthreads();
    }
    const int64_t before = threadIdx.x > 0 ? lds[threadIdx.x - 1] : 0;
    const int64_t total = lds[SCAN_THREADS - 1];
    __syncthreads();
    if (b < nblocks) partial[b] = carry > before ? carry : before;
    carry = carry > total ? carry : total;
  }
}

// pass 3: the repaired offsets (into `fixed`), the count of bad bags, the
// conditions a FATAL run reports
__global__ __launch_bounds__(SCAN_THREADS) void bounds_fix_offsets_kernel(
    const void* offsets, int is64, int64_t total_B, int64_t N, const int64_t* carry_in, int carry_is_prefix,
    int64_t* fixed, int mode, int64_t* warning, Status* status) {
  __shared__ int64_t lds[SCAN_THREADS];
  __shared__ int bad_count;
  if (threadIdx.x == 0) bad_count = 0;
  // what the blocks before this one leave: either pass 2 has made it (carry_is_prefix), or, with at most
  // SCAN_THREADS blocks, every block takes the maximum of the earlier blocks' maxima itself and pass 2 is not run
  int64_t carry;
  if (carry_is_prefix) {
    carry = carry_in[blockIdx.x];
  } else {
    carry = block_max(threadIdx.x < blockIdx.x ? carry_in[threadIdx.x] : 0, lds);
  }
  const int64_t base = (int64_t)blockIdx.x * SCAN_BLOCK + (int64_t)threadIdx.x * SCAN_ITEMS;
  int64_t v[SCAN_ITEMS];
  int64_t local = 0;
  for (int i = 0; i < SCAN_ITEMS; ++i) {
    const int64_t k = base + i;
    v[i] = k <= total_B ? clamped_offset(offsets, is64, k, total_B, N) : 0;
    local = v[i] > local ? v[i] : local;
  }
  // running maximum of the threads' local maxima before this thread: inside each wave through lane
  // shuffles, then over the 16 wave maxima (two workgroup barriers instead of twenty)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t incl = local;
  for (int step = 1; step < 64; step <<= 1) {
    const int64_t o = __shfl_up(incl, step, 64);
    if (lane >= step) incl = incl > o ? incl : o;
  }
  int64_t run = __shfl_up(incl, 1, 64); // exclusive inside the wave (values are >= 0)
  if (lane == 0) run = 0;
  __syncthreads(); // lds is free again (the carry above may have used it)
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  for (int w = 0; w < wave; ++w) run = run > lds[w] ? run : lds[w];
  run = run > carry ? run : carry;
  int bad = 0, err = 0;
  for (int i = 0; i < SCAN_ITEMS; ++i) {
    const int64_t k = base + i;
    if (k > total_B) break;
    run = v[i] > run ? v[i] : run; // repaired offsets[k]
    fixed[k] = run;
    if (k == total_B) {
      if (read_index(offsets, is64, total_B) != N) {
        ++bad; // "the last element in offsets is incorrect"
        err |= ERR_LENGTH_MISMATCH;
      }
    } else {
      // bag k: starts at the repaired offsets[k], ends at the original offsets[k + 1]
      const int64_t end = k + 1 == total_B ? N : read_index(offsets, is64, k + 1);
      const bool first_negative = k == 0 && read_index(offsets, is64, 0) < 0;
      // a first offset beyond num_indices is bad whatever follows it
      const bool first_high = k == 0 && read_index(offsets, is64, 0) > N;
      if (first_negative || first_high || run > end || end > N) {
        ++bad;
        err |= ERR_BAG_OVERRUN;
      }
    }
  }
  if (mode == 1 && bad) atomicAdd(&bad_count, bad);
  if (mode == 0 && err) atomicOr(&status->bits, err);
  __syncthreads();
  if (mode == 1 && threadIdx.x == 0 && bad_count) atomicAdd(reinterpret_cast<unsigned long long*>(warning), (unsigned long long)bad_count);
}

// pass 4: one group of 16 lanes per bag checks the bag's indices against its
// table's row count and (WARNING, IGNORE) writes the repairs back
constexpr int BAG_LANES = 16;
__global__ __launch_bounds__(256) void bounds_check_bags_kernel(
    const int64_t* rows_per_table, int32_t T, void* indices, void* offsets, int is64, int64_t total_B,
    int64_t B, const int32_t* B_offsets, const int64_t* fixed, int mode, int64_t* warning, Status* status) {
  __shared__ int bad_count;
  if (threadIdx.x == 0) bad_count = 0;
  __syncthreads();
  const int sub = threadIdx.x % BAG_LANES;
  const int64_t groups = (int64_t)gridDim.x * (blockDim.x / BAG_LANES);
  int bad = 0;
  for (int64_t bag = (int64_t)blockIdx.x * (blockDim.x / BAG_LANES) + threadIdx.x / BAG_LANES; bag < total_B; bag += groups) {
    int32_t t;
    if (B_offsets) {
      int32_t lo = 0, hi = T; // largest t with B_offsets[t] <= bag
      while (hi - lo > 1) {
        const int32_t mid = (lo + hi) / 2;
        if ((int64_t)B_offsets[mid] <= bag) lo = mid;
        else hi = mid;
      }
      t = lo;
    } else {
      t = (int32_t)(bag / B);
    }
    const int64_t num_rows = rows_per_table[t];
    const int64_t start = fixed[bag], end = fixed[bag + 1];
    for (int64_t i = start + sub; i < end; i += BAG_LANES) {
      const int64_t idx = read_index(indices, is64, i);
      if (idx == -1) continue; // pruned row
      if (idx < 0 || idx >= num_rows) {
        if (mode == 0) {
          atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
          atomicMin(&status->first_bad_pos, (unsigned long long)i);
        } else {
          ++bad;
          write_index(indices, is64, i, 0);
        }
      }
    }
    if (mode != 0 && sub == 0) {
      write_index(offsets, is64, bag, start);
      if (bag == total_B - 1) write_index(offsets, is64, total_B, end);
    }
  }
  if (mode == 1) {
    if (bad) atomicAdd(&bad_count, bad);
    __syncthreads();
    if (threadIdx.x == 0 && bad_count) atomicAdd(reinterpret_cast<unsigned long long*>(warning), (unsigned long long)bad_count);
  }
}

// MurmurHash3 finalizers, as the reference hashes sparse ids
// (embedding_forward_quantized_cpu_template.cpp:102-120)
__device__ __forceinline__ uint32_t pruned_hash(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}
__device__ __forceinline__ uint64_t pruned_hash(uint64_t k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return k;
}

// dense[i] = value of key indices[i] in its table's open-addressing map (linear
// probing, -1 = empty slot = not there), a copy for tables without a map
// (embedding_forward_quantized_cpu_template.cpp:524-603). One lane per index.
// A probe sequence ends after one trip round the table (the reference would
// not return from a full table that lacks the key).
template <typename index_t, typename hash_t>
__global__ __launch_bounds__(256) void pruned_hashmap_lookup_kernel(
    const index_t* indices, const index_t* offsets, const hash_t* hash_table, const int64_t* hash_table_offsets,
    int32_t B, index_t* dense) {
  using uidx_t = typename std::conditional<sizeof(index_t) == 8, uint64_t, uint32_t>::type;
  const int t = blockIdx.y;
  const int64_t table_start = hash_table_offsets[t];
  const int64_t capacity = hash_table_offsets[t + 1] - table_start;
  const int64_t is = offsets[(int64_t)t * B], ie = offsets[(int64_t)(t + 1) * B];
  for (int64_t i = is + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ie; i += (int64_t)gridDim.x * blockDim.x) {
    const index_t idx = indices[i];
    if (capacity == 0) {
      dense[i] = idx;
      continue;
    }
    int64_t slot;
    if (sizeof(index_t) == 8) slot = (int64_t)(pruned_hash((uint64_t)(uidx_t)idx) % (uint64_t)capacity);
    else slot = (int64_t)pruned_hash((uint32_t)(uidx_t)idx) % capacity;
    index_t out = (index_t)-1;
    for (int64_t probes = 0; probes < capacity; ++probes) {
      const hash_t* entry = hash_table + 2 * (table_start + slot);
      const hash_t key = entry[0];
      if (key == (hash_t)-1) break;
      if ((int64_t)key == (int64_t)idx) {
        out = (index_t)entry[1];
        break;
      }
      slot = slot + 1 == capacity ? 0 : slot + 1;
    }
    dense[i] = out;
  }
}

} // namespace

hipError_t launch_bounds_check(const int64_t* rows_per_table, int32_t T, void* indices, void* offsets, bool is64,
                               int64_t num_indices, int64_t total_B, int64_t B, const int32_t* B_offsets, int mode,
                               int64_t* warning, int64_t* fixed, int64_t* partial, Status* status, hipStream_t stream) {
  const int64_t n = total_B + 1;
  const int64_t nblocks = (n + SCAN_BLOCK - 1) / SCAN_BLOCK;
  hipLaunchKernelGGL(bounds_partial_max_kernel, dim3((unsigned)nblocks), dim3(SCAN_THREADS), 0, stream, offsets,
                     is64 ? 1 : 0, total_B, num_indices, partial, warning, mode);
  const int own_carry = nblocks <= SCAN_THREADS; // up to 4 M offsets: one launch less
  if (!own_carry) hipLaunchKernelGGL(bounds_carry_kernel, dim3(1), dim3(SCAN_THREADS), 0, stream, partial, nblocks);
  hipLaunchKernelGGL(bounds_fix_offsets_kernel, dim3((unsigned)nblocks), dim3(SCAN_THREADS), 0, stream, offsets,
                     is64 ? 1 : 0, total_B, num_indices, partial, own_carry ? 0 : 1, fixed, mode, warning, status);
  if (total_B > 0) {
    const int64_t per_block = 256 / BAG_LANES;
    int64_t blocks = (total_B + per_block - 1) / per_block;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(bounds_check_bags_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, rows_per_table, T,
                       indices, offsets, is64 ? 1 : 0, total_B, B, B_offsets, fixed, mode, warning, status);
  }
  return hipGetLastError();
}

int64_t bounds_check_partials(int64_t total_B) { return (total_B + 1 + SCAN_BLOCK - 1) / SCAN_BLOCK; }

hipError_t launch_pruned_hashmap_lookup(const void* indices, const void* offsets, bool idx64, const void* hash_table,
                                        bool hash64, const int64_t* hash_table_offsets, int32_t B, int32_t T,
                                        void* dense, hipStream_t stream) {
  if (T <= 0 || B <= 0) return hipSuccess;
  dim3 grid(64, (unsigned)T), block(256);
  if (idx64 && hash64)
    hipLaunchKernelGGL((pruned_hashmap_lookup_kernel<int64_t, int64_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int64_t*)hash_table, hash_table_offsets, B, (int64_t*)dense);
  else if (idx64)
    hipLaunchKernelGGL((pruned_hashmap_lookup_kernel<int64_t, int32_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int32_t*)hash_table, hash_table_offsets, B, (int64_t*)dense);
  else if (hash64)
    hipLaunchKernelGGL((pruned_hashmap_lookup_kernel<int32_t, int64_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int64_t*)hash_table, hash_table_offsets, B, (int32_t*)dense);
  else
    hipLaunchKernelGGL((pruned_hashmap_lookup_kernel<int32_t, int32_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int32_t*)hash_table, hash_table_offsets, B, (int32_t*)dense);
  return hipGetLastError();
}

} // namespace fbgemm_amd
