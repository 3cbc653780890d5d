// gfx950 kernels of embedding_bag_rowwise_prune, the step of the inference
// converter that drops the rows of a table whose importance indicator is at or
// below a threshold and leaves a remap array for the lookups
// (fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2836-2893, which ends in
// at::native::_rowwise_prune; caller:
// fbgemm_gpu/fbgemm_gpu/split_embedding_inference_converter.py:75-93).
//
// The reference walks the rows in order: a row is kept when its indicator
// (its absolute value with `abs`) exceeds the threshold, and, once the rows
// kept so far plus ALL rows still to come no longer exceed min_non_pruned_rows,
// every remaining row is kept. With P(i) the number of rows before i that pass
// the threshold test, f(i) = P(i) + rows - i never grows with i and drops by at
// most one per row, so the forced region is the suffix {i : f(i) <= min}, on
// which the running count of kept rows is i - max(rows - min, 0). One exclusive
// prefix sum of the threshold test therefore gives every row's new id:
//     remap[i] = P(i)                         threshold test passed, not forced
//              = i - max(rows - min, 0)       forced
//              = -1                           dropped
// and the result does not depend on how the GPU schedules the rows.
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

constexpr int PSCAN_THREADS = 1024;
constexpr int PSCAN_ITEMS = 4; // rows per thread
constexpr int PSCAN_BLOCK = PSCAN_THREADS * PSCAN_ITEMS;

// the reference compares the float indicator with the double threshold
__device__ __forceinline__ bool passes(const float* indicator, int64_t i, double threshold, int use_abs) {
  const float v = indicator[i];
  return (double)(use_abs ? __builtin_fabsf(v) : v) > threshold;
}

// compressed_indices_remap: position k of the index array stays when its row is not pruned.
// An index outside the mapping cannot be looked up: it is dropped and reported.
template <typename index_t>
__device__ __forceinline__ int32_t mapped_row(const index_t* indices, const int32_t* mapping, int64_t mapping_numel, int64_t k,
                                              Status* status) {
  const int64_t idx = (int64_t)indices[k];
  if (idx < 0 || idx >= mapping_numel) {
    atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
    atomicMin(&status->first_bad_pos, (unsigned long long)k);
    return -1;
  }
  return mapping[idx];
}

// inclusive sum over the workgroup's threads; returns this thread's inclusive value
__device__ __forceinline__ int64_t block_inclusive_sum(int64_t mine, int64_t* lds) {
  lds[threadIdx.x] = mine;
  __syncthreads();
  for (int step = 1; step < PSCAN_THREADS; step <<= 1) {
    const int64_t o = (int)threadIdx.x >= step ? lds[threadIdx.x - step] : 0;
    __syncthreads();
    lds[threadIdx.x] += o;
    __syncthreads();
  }
  const int64_t r = lds[threadIdx.x];
  __syncthreads();
  return r;
}

// pass 1: rows of every block of PSCAN_BLOCK rows that pass the threshold test
__global__ __launch_bounds__(PSCAN_THREADS) void prune_count_kernel(const float* indicator, int64_t rows, double threshold,
                                                                    int use_abs, int64_t* partial) {
  __shared__ int64_t lds[PSCAN_THREADS];
  const int64_t base = (int64_t)blockIdx.x * PSCAN_BLOCK + (int64_t)threadIdx.x * PSCAN_ITEMS;
  int64_t local = 0;
  for (int i = 0; i < PSCAN_ITEMS; ++i)
    if (base + i < rows && passes(indicator, base + i, threshold, use_abs)) ++local;
  const int64_t incl = block_inclusive_sum(local, lds);
  if (threadIdx.x == PSCAN_THREADS - 1) partial[blockIdx.x] = incl;
}

// pass 2 (one workgroup): partial[b] becomes the sum of all blocks before b
__global__ __launch_bounds__(PSCAN_THREADS) void prune_carry_kernel(int64_t* partial, int64_t nblocks) {
  __shared__ int64_t lds[PSCAN_THREADS];
  int64_t carry = 0;
  for (int64_t b0 = 0; b0 < nblocks; b0 += PSCAN_THREADS) {
    const int64_t b = b0 + threadIdx.x;
    const int64_t mine = b < nblocks ? partial[b] : 0;
    const int64_t incl = block_inclusive_sum(mine, lds);
    lds[threadIdx.x] = incl;
    __syncthreads();
    const int64_t total = lds[PSCAN_THREADS - 1];
    __syncthreads();
    if (b < nblocks) partial[b] = carry + incl - mine;
    carry += total;
  }
}

// pass 3: the remap array and the number of rows kept
template <typename index_t>
__global__ __launch_bounds__(PSCAN_THREADS) void prune_remap_kernel(const float* indicator, int64_t rows, double threshold,
                                                                    int use_abs, int64_t min_rows, const int64_t* carry_in,
                                                                    index_t* remap, int64_t* num_kept) {
  __shared__ int64_t lds[PSCAN_THREADS];
  const int64_t base = (int64_t)blockIdx.x * PSCAN_BLOCK + (int64_t)threadIdx.x * PSCAN_ITEMS;
  bool pass[PSCAN_ITEMS];
  int64_t local = 0;
  for (int i = 0; i < PSCAN_ITEMS; ++i) {
    pass[i] = base + i < rows && passes(indicator, base + i, threshold, use_abs);
    local += pass[i] ? 1 : 0;
  }
  const int64_t incl = block_inclusive_sum(local, lds);
  int64_t before = carry_in[blockIdx.x] + incl - local; // P(base)
  const int64_t shift = rows > min_rows ? rows - min_rows : 0;
  for (int i = 0; i < PSCAN_ITEMS; ++i) {
    const int64_t r = base + i;
    if (r >= rows) break;
    const bool forced = before + (rows - r) <= min_rows;
    const bool keep = pass[i] || forced;
    const int64_t id = forced ? r - shift : before;
    remap[r] = keep ? (index_t)id : (index_t)-1;
    if (r == rows - 1) *num_kept = id + (keep ? 1 : 0);
    before += pass[i] ? 1 : 0;
  }
}

// out[remap[r]] = in[r] for the rows that stay; `lpr` lanes per row, 16 bytes
// per lane and step where the buffers allow it
template <typename index_t>
__global__ __launch_bounds__(256) void prune_gather_kernel(const uint8_t* in, int64_t rows, int64_t row_bytes, const index_t* remap,
                                                           uint8_t* out, int64_t out_rows, int lpr, int vec) {
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int per_wave = 64 / lpr;
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t ngroups = (rows + per_wave - 1) / per_wave;
  for (int64_t g = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); g < ngroups; g += nwaves) {
    const int64_t r = g * per_wave + lane / lpr;
    if (r >= rows) continue;
    const int64_t to = (int64_t)remap[r];
    if (to < 0 || to >= out_rows) continue;
    const uint8_t* src = in + r * row_bytes;
    uint8_t* dst = out + to * row_bytes;
    if (vec) {
      for (int64_t b = (int64_t)sub * 16; b < row_bytes; b += (int64_t)lpr * 16)
      {
        const uint4 q = *reinterpret_cast<const uint4*>(src + b);
        stream_store16(dst + b, q.x, q.y, q.z, q.w);
      }
    } else {
      for (int64_t b = sub; b < row_bytes; b += lpr) dst[b] = src[b];
    }
  }
}

// ---- compressed_indices_remap ----------------------------------------------
// src/RefImplementations.cc:2308-2333 (AVX-512 twin: src/EmbeddingSpMDMAvx512.cc):
// the entries of the bags whose row is pruned (mapping[index] == -1) are dropped,
// the others are replaced by their physical row and moved up, per-sample weights
// move with them, and out_offsets[i] counts the entries that stay before bag i
// (out_offsets[0] = offsets[0], as the reference writes it). With offsets that
// do not decrease the reference visits positions offsets[0] .. offsets[last]-1
// in order, so the new position of an entry is the number of entries that stay
// before it: one exclusive prefix sum.

// pass 1: entries of every block of PSCAN_BLOCK positions that stay
template <typename index_t>
__global__ __launch_bounds__(PSCAN_THREADS) void remap_count_kernel(const index_t* indices, const int32_t* mapping,
                                                                    int64_t mapping_numel, int64_t first, int64_t n,
                                                                    int64_t* partial, int32_t* mapped, Status* status) {
  __shared__ int64_t lds[PSCAN_THREADS];
  const int64_t base = (int64_t)blockIdx.x * PSCAN_BLOCK + (int64_t)threadIdx.x * PSCAN_ITEMS;
  int64_t local = 0;
  for (int i = 0; i < PSCAN_ITEMS; ++i) {
    if (base + i < n) {
      // the gather through the mapping is made once: pass 3 reads the rows back in order
      const int32_t row = mapped_row(indices, mapping, mapping_numel, first + base + i, status);
      mapped[base + i] = row;
      if (row != -1) ++local;
    }
  }
  const int64_t incl = block_inclusive_sum(local, lds);
  if (threadIdx.x == PSCAN_THREADS - 1) partial[blockIdx.x] = incl;
}

// pass 3: move the entries; before[k] = entries that stay in front of position first + k (k = 0 .. n)
template <typename index_t>
__global__ __launch_bounds__(PSCAN_THREADS) void remap_move_kernel(const int32_t* mapped, const float* weights, int64_t first,
                                                                   int64_t n, const int64_t* carry_in, index_t* out_indices,
                                                                   float* out_weights, int64_t* before_out) {
  __shared__ int64_t lds[PSCAN_THREADS];
  const int64_t base = (int64_t)blockIdx.x * PSCAN_BLOCK + (int64_t)threadIdx.x * PSCAN_ITEMS;
  int32_t row[PSCAN_ITEMS];
  int64_t local = 0;
  for (int i = 0; i < PSCAN_ITEMS; ++i) {
    row[i] = base + i < n ? mapped[base + i] : -1;
    local += row[i] != -1 ? 1 : 0;
  }
  const int64_t incl = block_inclusive_sum(local, lds);
  int64_t before = carry_in[blockIdx.x] + incl - local;
  for (int i = 0; i < PSCAN_ITEMS; ++i) {
    const int64_t k = base + i;
    if (k > n) break;
    before_out[k] = before; // k == n: the total
    if (k == n) break;
    if (row[i] != -1) {
      out_indices[before] = (index_t)row[i];
      if (weights) out_weights[before] = weights[first + k];
      ++before;
    }
  }
}

template <typename index_t>
__global__ __launch_bounds__(256) void remap_offsets_kernel(const index_t* offsets, int64_t offsets_numel, int64_t first,
                                                            int64_t n, const int64_t* before, index_t* out_offsets) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= offsets_numel) return;
  if (i == 0) {
    out_offsets[0] = offsets[0];
    return;
  }
  int64_t k = (int64_t)offsets[i] - first;
  k = k < 0 ? 0 : (k > n ? n : k);
  out_offsets[i] = (index_t)before[k];
}

} // namespace

int64_t prune_partials(int64_t rows) { return (rows + PSCAN_BLOCK - 1) / PSCAN_BLOCK; }

hipError_t launch_prune_map(const float* indicator, int64_t rows, double threshold, int use_abs, int64_t min_rows,
                            bool idx64, void* remap, int64_t* num_kept, int64_t* partial, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  const int64_t nblocks = prune_partials(rows);
  hipLaunchKernelGGL(prune_count_kernel, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, indicator, rows, threshold,
                     use_abs, partial);
  hipLaunchKernelGGL(prune_carry_kernel, dim3(1), dim3(PSCAN_THREADS), 0, stream, partial, nblocks);
  if (idx64)
    hipLaunchKernelGGL(prune_remap_kernel<int64_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, indicator, rows,
                       threshold, use_abs, min_rows, partial, (int64_t*)remap, num_kept);
  else
    hipLaunchKernelGGL(prune_remap_kernel<int32_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, indicator, rows,
                       threshold, use_abs, min_rows, partial, (int32_t*)remap, num_kept);
  return hipGetLastError();
}

hipError_t launch_prune_gather(const void* in, int64_t rows, int64_t row_bytes, const void* remap, bool idx64, void* out,
                               int64_t out_rows, hipStream_t stream) {
  if (rows <= 0 || row_bytes <= 0) return hipSuccess;
  const int vec = row_bytes % 16 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
  const int64_t units = vec ? row_bytes / 16 : row_bytes;
  int lpr = 1;
  while (lpr < 64 && lpr < units) lpr <<= 1;
  const int64_t per_block = 4 * (64 / lpr);
  int64_t blocks = (rows + per_block - 1) / per_block;
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (idx64)
    hipLaunchKernelGGL(prune_gather_kernel<int64_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)in, rows,
                       row_bytes, (const int64_t*)remap, (uint8_t*)out, out_rows, lpr, vec);
  else
    hipLaunchKernelGGL(prune_gather_kernel<int32_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)in, rows,
                       row_bytes, (const int32_t*)remap, (uint8_t*)out, out_rows, lpr, vec);
  return hipGetLastError();
}

// n = offsets[last] - offsets[0] positions starting at `first` = offsets[0]; `before` holds n + 1 entries,
// `partial` prune_partials(n + 1), `mapped` n.
hipError_t launch_compressed_indices_remap(const void* indices, bool idx64, const int32_t* mapping, int64_t mapping_numel,
                                           const void* offsets, int64_t offsets_numel, const float* weights, int64_t first,
                                           int64_t n, void* out_indices, void* out_offsets, float* out_weights,
                                           int64_t* before, int64_t* partial, int32_t* mapped, Status* status,
                                           hipStream_t stream) {
  const int64_t nblocks = prune_partials(n + 1);
  const unsigned oblocks = (unsigned)((offsets_numel + 255) / 256);
  if (idx64) {
    hipLaunchKernelGGL(remap_count_kernel<int64_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, (const int64_t*)indices,
                       mapping, mapping_numel, first, n, partial, mapped, status);
    hipLaunchKernelGGL(prune_carry_kernel, dim3(1), dim3(PSCAN_THREADS), 0, stream, partial, nblocks);
    hipLaunchKernelGGL(remap_move_kernel<int64_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, (const int32_t*)mapped,
                       weights, first, n, partial, (int64_t*)out_indices, out_weights, before);
    hipLaunchKernelGGL(remap_offsets_kernel<int64_t>, dim3(oblocks), dim3(256), 0, stream, (const int64_t*)offsets, offsets_numel,
                       first, n, before, (int64_t*)out_offsets);
  } else {
    hipLaunchKernelGGL(remap_count_kernel<int32_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, (const int32_t*)indices,
                       mapping, mapping_numel, first, n, partial, mapped, status);
    hipLaunchKernelGGL(prune_carry_kernel, dim3(1), dim3(PSCAN_THREADS), 0, stream, partial, nblocks);
    hipLaunchKernelGGL(remap_move_kernel<int32_t>, dim3((unsigned)nblocks), dim3(PSCAN_THREADS), 0, stream, (const int32_t*)mapped,
                       weights, first, n, partial, (int32_t*)out_indices, out_weights, before);
    hipLaunchKernelGGL(remap_offsets_kernel<int32_t>, dim3(oblocks), dim3(256), 0, stream, (const int32_t*)offsets, offsets_numel,
                       first, n, before, (int32_t*)out_offsets);
  }
  return hipGetLastError();
}

} // namespace fbgemm_amd
