// gfx950 kernels that write one output row per index: the table-batched
// forward without pooling (PoolingMode.NONE, "sequence" output) and, at the end
// of the file, the no_bag mode of the single-table kernels.
//
// What the reference's CPU operator does for this mode
// (fbgemm_gpu/codegen/inference/embedding_forward_quantized_cpu_template.cpp:283-296,390-420):
// every index is a bag of length one, so row i of the [total_L, D] output is
//     out[i][j] = convert(fma(1.0f * scale, q[j], 0.0f + 1.0f * bias))     (quantised rows)
//     out[i][j] = convert(fma(1.0f, x[j], 0.0f))                           (fp16 / fp32 rows)
// of row indices[i] of the table position i belongs to (the table whose slice
// of `offsets` holds i); an index of -1 (pruned row) leaves zeros. With an
// int8 or int4 output type the row's bytes (fp16 scale/bias first, then the
// elements) are copied as they are (src/RefImplementations.cc:1235-1253,
// 1466-1484): all tables then hold rows of that type.
//
// `lpr` lanes share an output row; a lane turns runs of 4 elements into one
// store. The table of a position is found by bisection over the T + 1 table
// boundaries, which the workgroup keeps in LDS.
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

constexpr int SRUN = 8; // columns per lane and step: a whole number of bytes for every row type
constexpr int MAX_LDS_TABLES = 1024; // boundaries kept in LDS; beyond that they are read from memory

__device__ __forceinline__ float s_bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t s_float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float s_half_to_float(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t s_to_half(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
__device__ __forceinline__ uint16_t s_to_bf16(float f) { return (uint16_t)((s_float_to_bits(f) + 0x8000u) >> 16); }

__device__ __forceinline__ int64_t s_read(const void* p, bool is64, int64_t i) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}

__device__ __forceinline__ int s_type_bits(int ty) {
  return ty == ST_FP32 ? 32 : (ty == ST_FP16 || ty == ST_BF16) ? 16 : (ty == ST_INT8 || ty == ST_FP8) ? 8 : ty == ST_INT4 ? 4 : 2;
}

// Copy `n_out` bytes of an output row: the first `n_in` from the table row, zeros after.
__device__ __forceinline__ void copy_row_bytes(const uint8_t* row, bool ok, int64_t n_in, int64_t n_out, uint8_t* orow,
                                               int sub, int lpr) {
  for (int64_t b0 = (int64_t)sub * 4; b0 < n_out; b0 += (int64_t)lpr * 4) {
    uint32_t v = 0;
    if (ok && b0 + 4 <= n_in && (reinterpret_cast<uintptr_t>(row + b0) & 3) == 0) v = *reinterpret_cast<const uint32_t*>(row + b0);
    else if (ok) for (int k = 0; k < 4; ++k) if (b0 + k < n_in) v |= (uint32_t)row[b0 + k] << (8 * k);
    if (b0 + 4 <= n_out && (reinterpret_cast<uintptr_t>(orow + b0) & 3) == 0) *reinterpret_cast<uint32_t*>(orow + b0) = v;
    else for (int k = 0; k < 4; ++k) if (b0 + k < n_out) orow[b0 + k] = (uint8_t)(v >> (8 * k));
  }
}

// dword-aligned groups of words: rows sit on 4-byte boundaries at best, which is all a wide load needs
struct __attribute__((aligned(4))) Words4 { uint32_t v[4]; };
struct __attribute__((aligned(4))) Words2 { uint32_t v[2]; };

// The bytes [b0, b0 + nbytes) of a row (nbytes <= 32) into w[], little end first:
// whole dwords where the address allows it, single bytes otherwise and at the tail.
__device__ __forceinline__ void load_run_bytes(const uint8_t* p, int nbytes, uint32_t (&w)[8]) {
  const bool a4 = (reinterpret_cast<uintptr_t>(p) & 3) == 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t v = 0;
    if (i * 4 + 4 <= nbytes && a4) {
      v = *reinterpret_cast<const uint32_t*>(p + i * 4);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (i * 4 + k < nbytes) v |= (uint32_t)p[i * 4 + k] << (8 * k);
    }
    w[i] = v;
  }
}

// One output row of D columns from one table row, as a bag of one with weight w:
//   quantised rows  out[j] = convert(fma(w * scale, q[j], 0 + w * bias))
//   plain rows      out[j] = convert(fma(w, x[j], 0))
// `lpr` lanes share the row, lane `sub` takes runs of SRUN columns (one to eight
// dword loads, one or two 16-byte stores). A row that is not there (!ok) gives
// zeros; columns past the table's own width give zeros. TY is the row type, so
// that widths and bit positions are constants.
template <int TY>
__device__ __forceinline__ void emit_row_t(const TableDesc& d, const uint8_t* row, bool ok, float w, int D, int out_ty,
                                           uint8_t* orow, int sub, int lpr, int fp8_shift, float fp8_mult) {
  constexpr int bits = TY == ST_FP32 ? 32 : (TY == ST_FP16 || TY == ST_BF16) ? 16 : (TY == ST_INT8 || TY == ST_FP8) ? 8 : TY == ST_INT4 ? 4 : 2;
  constexpr bool quant = TY == ST_INT8 || TY == ST_INT4 || TY == ST_INT2;
  constexpr int run_bytes = (SRUN * bits) >> 3; // 2 .. 32
  float scale = w, bias = 0.0f;
  if (quant && ok) {
    const uint8_t* ph = row + d.sb_off;
    if (d.sb_fp32) {
      uint32_t h[2];
      for (int k = 0; k < 2; ++k) {
        const uint8_t* q = ph + 4 * k;
        if ((reinterpret_cast<uintptr_t>(q) & 3) == 0) h[k] = *reinterpret_cast<const uint32_t*>(q);
        else h[k] = q[0] | (q[1] << 8) | (q[2] << 16) | ((uint32_t)q[3] << 24);
      }
      scale = w * s_bits_to_float(h[0]);
      bias = w * s_bits_to_float(h[1]);
    } else {
      uint32_t h;
      if ((reinterpret_cast<uintptr_t>(ph) & 3) == 0) h = *reinterpret_cast<const uint32_t*>(ph);
      else h = ph[0] | (ph[1] << 8) | (ph[2] << 16) | ((uint32_t)ph[3] << 24);
      scale = w * s_half_to_float((uint16_t)h);
      bias = w * s_half_to_float((uint16_t)(h >> 16));
    }
  }
  const uint8_t* data = row + d.data_off;
  const int Dt = d.D < D ? d.D : D;
  const int data_bytes = (Dt * bits + 7) >> 3; // the bytes of the row that hold columns < Dt
  for (int j0 = sub * SRUN; j0 < D; j0 += lpr * SRUN) {
    // SRUN is a multiple of 8 / bits for every type, so a run starts on a byte
    const int b0 = (j0 * bits) >> 3;
    uint32_t raw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[i] = 0;
    const uint8_t* p = data + b0;
    if (ok && b0 + run_bytes <= data_bytes && (reinterpret_cast<uintptr_t>(p) & 3) == 0 && run_bytes >= 4) {
      // a whole run on a dword boundary: the common case
      if constexpr (run_bytes == 32) {
        const Words4 a = *reinterpret_cast<const Words4*>(p), b = *reinterpret_cast<const Words4*>(p + 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) { raw[i] = a.v[i]; raw[4 + i] = b.v[i]; }
      } else if constexpr (run_bytes == 16) {
        const Words4 a = *reinterpret_cast<const Words4*>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) raw[i] = a.v[i];
      } else if constexpr (run_bytes == 8) {
        const Words2 a = *reinterpret_cast<const Words2*>(p);
        raw[0] = a.v[0]; raw[1] = a.v[1];
      } else {
        raw[0] = *reinterpret_cast<const uint32_t*>(p);
      }
    } else if (ok && b0 < data_bytes) {
      int nb = data_bytes - b0;
      load_run_bytes(p, nb < run_bytes ? nb : run_bytes, raw);
    }
    float v[SRUN];
#pragma unroll
    for (int k = 0; k < SRUN; ++k) {
      float x = 0.0f;
      if (ok && j0 + k < Dt) {
        if constexpr (bits == 32) {
          x = __builtin_fmaf(w, s_bits_to_float(raw[k]), 0.0f);
        } else if constexpr (bits == 16) {
          const uint16_t u = (uint16_t)(raw[k >> 1] >> (16 * (k & 1)));
          x = __builtin_fmaf(w, TY == ST_BF16 ? s_bits_to_float((uint32_t)u << 16) : s_half_to_float(u), 0.0f);
        } else if constexpr (TY == ST_FP8) {
          // Float8ToFloat_ref (src/RefImplementations.cc:184-214), then the bag of one: fma(w, x, 0)
          const uint32_t b = (raw[k >> 2] >> (8 * (k & 3))) & 0xffu;
          const float mag = s_bits_to_float((b & 0x7fu) << fp8_shift) * fp8_mult;
          x = __builtin_fmaf(w, s_bits_to_float(s_float_to_bits(mag) | ((b & 0x80u) << 24)), 0.0f);
        } else {
          const uint32_t q = (raw[(k * bits) >> 5] >> ((k * bits) & 31)) & ((1u << bits) - 1);
          x = __builtin_fmaf(scale, (float)q, 0.0f + bias);
        }
      }
      v[k] = x;
    }
    const int n = D - j0 < SRUN ? D - j0 : SRUN;
    if (out_ty == ST_FP32) {
      float* op = reinterpret_cast<float*>(orow) + j0;
      if (n == SRUN && (reinterpret_cast<uintptr_t>(op) & 15) == 0) {
#pragma unroll
        for (int k = 0; k < SRUN; k += 4) *reinterpret_cast<float4*>(op + k) = make_float4(v[k], v[k + 1], v[k + 2], v[k + 3]);
      } else {
        for (int k = 0; k < n; ++k) op[k] = v[k];
      }
    } else {
      uint32_t h[SRUN / 2];
#pragma unroll
      for (int k = 0; k < SRUN; k += 2) {
        const uint32_t lo = out_ty == ST_FP16 ? s_to_half(v[k]) : s_to_bf16(v[k]);
        const uint32_t hi = out_ty == ST_FP16 ? s_to_half(v[k + 1]) : s_to_bf16(v[k + 1]);
        h[k >> 1] = lo | (hi << 16);
      }
      uint16_t* op = reinterpret_cast<uint16_t*>(orow) + j0;
      if (n == SRUN && (reinterpret_cast<uintptr_t>(op) & 15) == 0) {
        *reinterpret_cast<uint4*>(op) = make_uint4(h[0], h[1], h[2], h[3]);
      } else {
        for (int k = 0; k < n; ++k) op[k] = (uint16_t)(h[k >> 1] >> (16 * (k & 1)));
      }
    }
  }
}

__device__ __forceinline__ void emit_row(const TableDesc& d, const uint8_t* row, bool ok, float w, int D, int out_ty,
                                         uint8_t* orow, int sub, int lpr, int fp8_shift, float fp8_mult) {
  switch (d.ty) {
    case ST_INT4: emit_row_t<ST_INT4>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_INT8: emit_row_t<ST_INT8>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_FP16: emit_row_t<ST_FP16>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_INT2: emit_row_t<ST_INT2>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_FP32: emit_row_t<ST_FP32>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_BF16: emit_row_t<ST_BF16>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    case ST_FP8: emit_row_t<ST_FP8>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult); break;
    default: break;
  }
}

template <typename index_t>
__global__ __launch_bounds__(256) void sequence_lookup_kernel(
    const TableDesc* tables, const uint8_t* w0, const uint8_t* w1, const index_t* indices, const void* offsets,
    int off64, int32_t B, int32_t T, int64_t total_L, int32_t D, int32_t out_ty, void* out, int32_t lpr,
    int32_t fp8_shift, float fp8_mult, Status* status) {
  __shared__ int64_t bounds[MAX_LDS_TABLES + 1];
  const bool in_lds = T <= MAX_LDS_TABLES;
  if (in_lds) {
    for (int t = threadIdx.x; t <= T; t += blockDim.x) bounds[t] = s_read(offsets, off64, (int64_t)t * B);
  }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int per_wave = 64 / lpr;
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t ngroups = (total_L + per_wave - 1) / per_wave;
  const bool copy_rows = out_ty == ST_INT8 || out_ty == ST_INT4;
  // bytes of an output row
  const int64_t out_row_bytes = out_ty == ST_FP32 ? (int64_t)D * 4 : (out_ty == ST_FP16 || out_ty == ST_BF16) ? (int64_t)D * 2
      : out_ty == ST_INT8 ? (int64_t)D + 4 : (int64_t)(D + 8 + 1) / 2;
  // the table of position `pos`: the largest t with bounds[t] <= pos (empty tables
  // share a boundary: the last of them wins)
  auto table_of = [&](int64_t pos) -> int {
    int lo = 0, hi = T; // invariant: bounds[lo] <= pos < bounds[hi] once the input is well formed
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      const int64_t b = in_lds ? bounds[mid] : s_read(offsets, off64, (int64_t)mid * B);
      if (b <= pos) lo = mid;
      else hi = mid;
    }
    return lo;
  };
  // The index and the table descriptor of the NEXT group of positions are
  // fetched while the rows of the current one are in flight, so that a wave
  // waits for one memory round trip per group instead of two.
  int64_t g = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  int64_t pos = g * per_wave + lane / lpr;
  bool live = g < ngroups && pos < total_L;
  int64_t idx = live ? (int64_t)indices[pos] : 0;
  TableDesc d = tables[live ? table_of(pos) : 0];
  while (g < ngroups) {
    const int64_t g2 = g + nwaves;
    const int64_t pos2 = g2 * per_wave + lane / lpr;
    const bool live2 = g2 < ngroups && pos2 < total_L;
    const int64_t idx2 = live2 ? (int64_t)indices[pos2] : 0;
    const TableDesc d2 = tables[live2 ? table_of(pos2) : 0];
    if (live) {
      uint8_t* orow = reinterpret_cast<uint8_t*>(out) + pos * out_row_bytes;
      bool ok = true;
      if (idx == -1) {
        ok = false; // pruned row: zeros
      } else if (idx < 0 || idx >= d.num_rows) {
        if (sub == 0) {
          atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
          atomicMin(&status->first_bad_pos, (unsigned long long)pos);
        }
        ok = false;
      }
      const uint8_t* row = (d.placement ? w1 : w0) + d.weights_offset + (ok ? idx : 0) * d.row_stride;
      if (copy_rows) {
        // the row as it is stored: header, then elements (what fits the output row)
        const int64_t in_bytes = d.data_off + d.data_bytes;
        copy_row_bytes(row, ok, in_bytes < out_row_bytes ? in_bytes : out_row_bytes, out_row_bytes, orow, sub, lpr);
      } else {
        emit_row(d, row, ok, 1.0f, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult);
      }
    }
    g = g2;
    pos = pos2;
    live = live2;
    idx = idx2;
    d = d2;
  }
}

// The single-table kernels' no_bag mode (src/RefImplementations.cc:1235-1288,
// 1352-1376, 1466-1484): output row m comes from table row indices[m], scaled
// by weights[m] when weights are given; any index outside [0, num_rows) is an
// error (-1 included). copy_bytes > 0 selects the byte-copy outputs: that many
// bytes of the stored row go to the output row and the rest of it stays as it was.
template <typename index_t>
__global__ __launch_bounds__(256) void row_lookup_kernel(
    TableDesc d, const uint8_t* table, const index_t* indices, const float* weights, int64_t n, int32_t out_ty,
    void* out, int64_t out_stride_bytes, int64_t copy_bytes, int32_t lpr, int32_t fp8_shift, float fp8_mult,
    Status* status) {
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int per_wave = 64 / lpr;
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t ngroups = (n + per_wave - 1) / per_wave;
  // the index and weight of the next group are fetched while this group's rows are in flight
  int64_t g = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  int64_t pos = g * per_wave + lane / lpr;
  bool live = g < ngroups && pos < n;
  int64_t idx = live ? (int64_t)indices[pos] : 0;
  float w = (live && weights) ? weights[pos] : 1.0f;
  while (g < ngroups) {
    const int64_t g2 = g + nwaves;
    const int64_t pos2 = g2 * per_wave + lane / lpr;
    const bool live2 = g2 < ngroups && pos2 < n;
    const int64_t idx2 = live2 ? (int64_t)indices[pos2] : 0;
    const float w2 = (live2 && weights) ? weights[pos2] : 1.0f;
    if (live) {
      const bool ok = idx >= 0 && idx < d.num_rows;
      if (!ok && sub == 0) {
        atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
        atomicMin(&status->first_bad_pos, (unsigned long long)pos);
      }
      const uint8_t* row = table + (ok ? idx : 0) * d.row_stride;
      uint8_t* orow = reinterpret_cast<uint8_t*>(out) + pos * out_stride_bytes;
      if (copy_bytes > 0) {
        if (ok) copy_row_bytes(row, true, copy_bytes, copy_bytes, orow, sub, lpr);
      } else {
        emit_row(d, row, ok, w, d.D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult);
      }
    }
    g = g2;
    pos = pos2;
    live = live2;
    idx = idx2;
    w = w2;
  }
}

} // namespace

hipError_t launch_sequence_lookup(const TableDesc* tables, const uint8_t* w0, const uint8_t* w1, const void* indices,
                                  bool idx64, const void* offsets, int32_t B, int32_t T, int64_t total_L, int32_t D,
                                  int32_t out_ty, void* out, int32_t fp8_shift, float fp8_mult, Status* status,
                                  hipStream_t stream) {
  if (total_L <= 0 || D <= 0) return hipSuccess;
  const int64_t row_units = out_ty == ST_INT8 ? (D + 4 + 3) / 4 : out_ty == ST_INT4 ? ((D + 9) / 2 + 3) / 4 : (D + SRUN - 1) / SRUN;
  int lpr = 1;
  while (lpr < 64 && lpr < row_units) lpr <<= 1;
  const int64_t per_block = 4 * (64 / lpr);
  int64_t blocks = (total_L + per_block - 1) / per_block;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid((unsigned)blocks), block(256);
  if (idx64)
    hipLaunchKernelGGL(sequence_lookup_kernel<int64_t>, grid, block, 0, stream, tables, w0, w1, (const int64_t*)indices,
                       offsets, 1, B, T, total_L, D, out_ty, out, lpr, fp8_shift, fp8_mult, status);
  else
    hipLaunchKernelGGL(sequence_lookup_kernel<int32_t>, grid, block, 0, stream, tables, w0, w1, (const int32_t*)indices,
                       offsets, 0, B, T, total_L, D, out_ty, out, lpr, fp8_shift, fp8_mult, status);
  return hipGetLastError();
}

hipError_t launch_row_lookup(const TableDesc& d, const uint8_t* table, const void* indices, bool idx64,
                             const float* weights, int64_t n, int32_t out_ty, void* out, int64_t out_stride_bytes,
                             int64_t copy_bytes, int32_t fp8_shift, float fp8_mult, Status* status, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const int64_t row_units = copy_bytes > 0 ? (copy_bytes + 3) / 4 : (d.D + SRUN - 1) / SRUN;
  int lpr = 1;
  while (lpr < 64 && lpr < row_units) lpr <<= 1;
  const int64_t per_block = 4 * (64 / lpr);
  int64_t blocks = (n + per_block - 1) / per_block;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid((unsigned)blocks), block(256);
  if (idx64)
    hipLaunchKernelGGL(row_lookup_kernel<int64_t>, grid, block, 0, stream, d, table, (const int64_t*)indices, weights, n,
                       out_ty, out, out_stride_bytes, copy_bytes, lpr, fp8_shift, fp8_mult, status);
  else
    hipLaunchKernelGGL(row_lookup_kernel<int32_t>, grid, block, 0, stream, d, table, (const int32_t*)indices, weights, n,
                       out_ty, out, out_stride_bytes, copy_bytes, lpr, fp8_shift, fp8_mult, status);
  return hipGetLastError();
}

} // namespace fbgemm_amd
