// gfx950 kernels of the in-place row update of a table-batched weights buffer:
// emb_inplace_update (fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update.cu:28-101,207-282,
// CPU form embedding_inplace_update_cpu.cpp:25-70) and the remap of the rows to
// update through the pruning arrays, pruned_array_lookup_from_row_idx
// (embedding_inplace_update.cu:359-465, embedding_inplace_update_cpu.cpp:199-251).
//
// An update is (table, row, byte offset into update_weights); the padded row of
// that table is overwritten with the bytes found there. A power-of-two group of
// lanes (as many as the widest row has 16-byte chunks, at most 16) moves one
// row, sixteen bytes per lane and step when source, destination and row size
// allow, so a wave writes 4 to 64 rows at a time. Two updates of one row in the
// same call race (as they do in the reference's kernel; its CPU loop lets the
// last one win).
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

template <typename index_t>
__global__ __launch_bounds__(256) void inplace_update_kernel(
    const TableDesc* tables, int32_t T, uint8_t* w0, uint8_t* w1, const uint8_t* update, int64_t update_bytes,
    const int32_t* table_idx, const index_t* row_idx, const int64_t* update_offsets, int64_t n, int32_t lpr,
    Status* status) {
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int per_wave = 64 / lpr;
  const int64_t stride = (int64_t)gridDim.x * 4 * per_wave;
  int64_t u = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * per_wave + lane / lpr;
  // the (table, row, offset) triple of the next update is fetched while the bytes of this one move
  int32_t t = u < n ? table_idx[u] : 0;
  int64_t r = u < n ? (int64_t)row_idx[u] : -1;
  int64_t uoff = u < n ? update_offsets[u] : 0;
  while (u < n) {
    const int64_t u2 = u + stride;
    const int32_t t2 = u2 < n ? table_idx[u2] : 0;
    const int64_t r2 = u2 < n ? (int64_t)row_idx[u2] : -1;
    const int64_t uoff2 = u2 < n ? update_offsets[u2] : 0;
    if (r != -1) { // a pruned row has no storage
      bool bad = t < 0 || t >= T;
      int64_t bytes = 0, woff = 0;
      int32_t placement = 0;
      if (!bad) {
        const TableDesc* d = tables + t;
        bytes = d->row_stride;
        woff = d->weights_offset;
        placement = d->placement;
        bad = r < 0 || r >= d->num_rows;
      }
      if (bad) {
        if (sub == 0 && status) {
          atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
          atomicMin(&status->first_bad_pos, (unsigned long long)u);
        }
      } else if (uoff < 0 || uoff + bytes > update_bytes) {
        if (sub == 0 && status) atomicOr(&status->bits, ERR_BAG_OVERRUN);
      } else {
        const uint8_t* src = update + uoff;
        uint8_t* dst = (placement ? w1 : w0) + woff + r * bytes;
        if ((((uintptr_t)src | (uintptr_t)dst | (uintptr_t)bytes) & 15) == 0) {
          const uint4* s16 = reinterpret_cast<const uint4*>(src);
          uint4* d16 = reinterpret_cast<uint4*>(dst);
          for (int64_t c = sub; c * 16 < bytes; c += lpr) d16[c] = s16[c];
        } else {
          for (int64_t b = sub; b < bytes; b += lpr) dst[b] = src[b];
        }
      }
    }
    u = u2, t = t2, r = r2, uoff = uoff2;
  }
}

// dense[i] = remap[remap_offsets[t_i] + row_i] where table t_i owns a mapping,
// row_i otherwise. A row outside its mapping, or a table outside [0, T), yields
// -1 (the reference reads out of bounds there).
template <typename index_t, typename remap_t>
__global__ __launch_bounds__(256) void remap_row_idx_kernel(const index_t* rows, const int32_t* table_idx, const remap_t* remap,
                                                            const int64_t* remap_offsets, int32_t T, int64_t n,
                                                            index_t* dense) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int32_t t = table_idx[i];
    index_t v = rows[i];
    if (t < 0 || t >= T) {
      v = (index_t)-1;
    } else {
      const int64_t rs = remap_offsets[t], cap = remap_offsets[t + 1] - rs;
      if (cap > 0) v = (v >= 0 && (int64_t)v < cap) ? (index_t)remap[rs + v] : (index_t)-1;
    }
    dense[i] = v;
  }
}

} // namespace

hipError_t launch_inplace_update(const TableDesc* tables, int32_t T, uint8_t* w0, uint8_t* w1, const uint8_t* update,
                                 int64_t update_bytes, const int32_t* table_idx, const void* row_idx, bool idx64,
                                 const int64_t* update_offsets, int64_t n, int64_t max_row_bytes, Status* status,
                                 hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  int lpr = 1;
  while (lpr < 16 && lpr * 16 < max_row_bytes) lpr <<= 1;
  const int64_t per_block = 4 * (64 / lpr);
  int64_t blocks = (n + per_block - 1) / per_block;
  if (blocks > 256 * 16) blocks = 256 * 16;
  const dim3 grid((unsigned)blocks), block(256);
  if (idx64)
    hipLaunchKernelGGL(inplace_update_kernel<int64_t>, grid, block, 0, stream, tables, T, w0, w1, update, update_bytes,
                       table_idx, (const int64_t*)row_idx, update_offsets, n, lpr, status);
  else
    hipLaunchKernelGGL(inplace_update_kernel<int32_t>, grid, block, 0, stream, tables, T, w0, w1, update, update_bytes,
                       table_idx, (const int32_t*)row_idx, update_offsets, n, lpr, status);
  return hipGetLastError();
}

hipError_t launch_remap_row_idx(const void* rows, bool idx64, const int32_t* table_idx, const void* remap, bool remap64,
                                const int64_t* remap_offsets, int32_t T, int64_t n, void* dense, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  const dim3 grid((unsigned)blocks), block(256);
  if (idx64 && remap64)
    hipLaunchKernelGGL((remap_row_idx_kernel<int64_t, int64_t>), grid, block, 0, stream, (const int64_t*)rows, table_idx,
                       (const int64_t*)remap, remap_offsets, T, n, (int64_t*)dense);
  else if (idx64)
    hipLaunchKernelGGL((remap_row_idx_kernel<int64_t, int32_t>), grid, block, 0, stream, (const int64_t*)rows, table_idx,
                       (const int32_t*)remap, remap_offsets, T, n, (int64_t*)dense);
  else if (remap64)
    hipLaunchKernelGGL((remap_row_idx_kernel<int32_t, int64_t>), grid, block, 0, stream, (const int32_t*)rows, table_idx,
                       (const int64_t*)remap, remap_offsets, T, n, (int32_t*)dense);
  else
    hipLaunchKernelGGL((remap_row_idx_kernel<int32_t, int32_t>), grid, block, 0, stream, (const int32_t*)rows, table_idx,
                       (const int32_t*)remap, remap_offsets, T, n, (int32_t*)dense);
  return hipGetLastError();
}

} // namespace fbgemm_amd
