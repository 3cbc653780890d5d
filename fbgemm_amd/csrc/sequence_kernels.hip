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
// `lpr` lanes share an output row; a lane turns runs of 8 elements into one or
// two 16-byte stores, and has the loads of four rows in flight before it decodes
// the first (one row at a time leaves a wave with 256 bytes outstanding, far
// too little to cover the latency of random rows). The table of a position is
// found by bisection over the T + 1 table boundaries, which the workgroup keeps
// in LDS.
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
    if (b0 + 4 <= n_out && (reinterpret_cast<uintptr_t>(orow + b0) & 3) == 0) stream_store4(orow + b0, v);
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
// that widths and bit positions are constants. The work is cut in three pieces
// (header load, run load, decode and store) so that a caller can have the loads
// of several rows in flight before it decodes the first.
template <int TY>
struct RowTraits {
  static constexpr int bits = TY == ST_FP32 ? 32 : (TY == ST_FP16 || TY == ST_BF16) ? 16 : (TY == ST_INT8 || TY == ST_FP8) ? 8 : TY == ST_INT4 ? 4 : 2;
  static constexpr bool quant = TY == ST_INT8 || TY == ST_INT4 || TY == ST_INT2;
  static constexpr int run_bytes = (SRUN * bits) >> 3; // 2 .. 32
};

// The (scale, bias) words of a quantised row as stored: two fp32 patterns, or two halfs in hdr[0].
template <int TY>
__device__ __forceinline__ void load_header_t(const TableDesc& d, const uint8_t* row, bool ok, uint32_t (&hdr)[2]) {
  hdr[0] = hdr[1] = 0;
  if (RowTraits<TY>::quant && ok) {
    const uint8_t* ph = row + d.sb_off;
    if (d.sb_fp32) {
      for (int k = 0; k < 2; ++k) {
        const uint8_t* q = ph + 4 * k;
        if ((reinterpret_cast<uintptr_t>(q) & 3) == 0) hdr[k] = *reinterpret_cast<const uint32_t*>(q);
        else hdr[k] = q[0] | (q[1] << 8) | (q[2] << 16) | ((uint32_t)q[3] << 24);
      }
    } else {
      if ((reinterpret_cast<uintptr_t>(ph) & 3) == 0) hdr[0] = *reinterpret_cast<const uint32_t*>(ph);
      else hdr[0] = ph[0] | (ph[1] << 8) | (ph[2] << 16) | ((uint32_t)ph[3] << 24);
    }
  }
}

// The stored bytes of the run of SRUN columns that starts at column j0 (zeros where the row has none).
template <int TY>
__device__ __forceinline__ void load_run_t(const uint8_t* data, bool ok, int data_bytes, int j0, uint32_t (&raw)[8]) {
  constexpr int bits = RowTraits<TY>::bits;
  constexpr int run_bytes = RowTraits<TY>::run_bytes;
  // SRUN is a multiple of 8 / bits for every type, so a run starts on a byte
  const int b0 = (j0 * bits) >> 3;
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
}

// Columns [j0, j0 + SRUN) of the output row from the stored bytes of their run.
template <int TY>
__device__ __forceinline__ void decode_store_t(const uint32_t (&raw)[8], bool ok, float w, float scale, float bias, int j0, int Dt,
                                               int D, int out_ty, uint8_t* orow, int fp8_shift, float fp8_mult) {
  constexpr int bits = RowTraits<TY>::bits;
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
      for (int k = 0; k < SRUN; k += 4) stream_store16(op + k, v[k], v[k + 1], v[k + 2], v[k + 3]);
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
      stream_store16(op, h[0], h[1], h[2], h[3]);
    } else {
      for (int k = 0; k < n; ++k) op[k] = (uint16_t)(h[k >> 1] >> (16 * (k & 1)));
    }
  }
}

// The row from its header words and the stored bytes of this lane's first run
// (already loaded); the runs of further passes, when the row is wider than
// lpr * SRUN columns, are loaded here.
template <int TY>
__device__ __forceinline__ void finish_row_t(const TableDesc& d, const uint8_t* row, bool ok, float w, int D, int out_ty,
                                             uint8_t* orow, int sub, int lpr, int fp8_shift, float fp8_mult,
                                             const uint32_t (&hdr)[2], uint32_t (&raw)[8]) {
  constexpr int bits = RowTraits<TY>::bits;
  float scale = w, bias = 0.0f;
  if (RowTraits<TY>::quant && ok) {
    if (d.sb_fp32) {
      scale = w * s_bits_to_float(hdr[0]);
      bias = w * s_bits_to_float(hdr[1]);
    } else {
      scale = w * s_half_to_float((uint16_t)hdr[0]);
      bias = w * s_half_to_float((uint16_t)(hdr[0] >> 16));
    }
  }
  const uint8_t* data = row + d.data_off;
  const int Dt = d.D < D ? d.D : D;
  const int data_bytes = (Dt * bits + 7) >> 3; // the bytes of the row that hold columns < Dt
  int j0 = sub * SRUN;
  if (j0 < D) decode_store_t<TY>(raw, ok, w, scale, bias, j0, Dt, D, out_ty, orow, fp8_shift, fp8_mult);
  for (j0 += lpr * SRUN; j0 < D; j0 += lpr * SRUN) {
    load_run_t<TY>(data, ok, data_bytes, j0, raw);
    decode_store_t<TY>(raw, ok, w, scale, bias, j0, Dt, D, out_ty, orow, fp8_shift, fp8_mult);
  }
}

// header and first run of this lane: loads only, nothing waits for them here
template <int TY>
__device__ __forceinline__ void load_row_t(const TableDesc& d, const uint8_t* row, bool ok, int D, int sub, uint32_t (&hdr)[2],
                                           uint32_t (&raw)[8]) {
  load_header_t<TY>(d, row, ok, hdr);
  const int Dt = d.D < D ? d.D : D;
  const int j0 = sub * SRUN;
  if (j0 < D) {
    load_run_t<TY>(row + d.data_off, ok, (Dt * RowTraits<TY>::bits + 7) >> 3, j0, raw);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[i] = 0;
  }
}

#define FBGEMM_AMD_ROW_TYPE_SWITCH(ty, CALL)        \
  switch (ty) {                                     \
    case ST_INT4: { constexpr int TY = ST_INT4; CALL; } break; \
    case ST_INT8: { constexpr int TY = ST_INT8; CALL; } break; \
    case ST_FP16: { constexpr int TY = ST_FP16; CALL; } break; \
    case ST_INT2: { constexpr int TY = ST_INT2; CALL; } break; \
    case ST_FP32: { constexpr int TY = ST_FP32; CALL; } break; \
    case ST_BF16: { constexpr int TY = ST_BF16; CALL; } break; \
    case ST_FP8: { constexpr int TY = ST_FP8; CALL; } break;   \
    default: break;                                 \
  }

constexpr int SEQ_ROWS = 4; // rows a group of lanes has in flight at a time

// SEQ_ROWS rows of one table (the first `live_rows` of them exist), output rows
// `orow_step` bytes apart, for a lane whose run is a whole run inside every row
// and sits, like the headers, on a dword boundary (the caller checks): every load
// is issued before the first row is decoded.
template <int TY>
__device__ __forceinline__ void rows_fast_t(const TableDesc& d, const uint8_t* const (&row)[SEQ_ROWS], const bool (&ok)[SEQ_ROWS],
                                            int live_rows, int D, int out_ty, uint8_t* orow0, int64_t orow_step, int sub,
                                            int fp8_shift, float fp8_mult) {
  constexpr int bits = RowTraits<TY>::bits;
  constexpr int run_bytes = RowTraits<TY>::run_bytes;
  constexpr int words = run_bytes >= 4 ? run_bytes / 4 : 1;
  const int j0 = sub * SRUN;
  const int off = d.data_off + ((j0 * bits) >> 3);
  // rows in flight at a time: 32 bytes per lane for the wide types, all SEQ_ROWS rows for the narrow ones
  constexpr int BATCH = words >= 8 ? 1 : words >= 4 ? 2 : SEQ_ROWS;
  const int Dt = d.D < D ? d.D : D;
#pragma unroll
  for (int k0 = 0; k0 < SEQ_ROWS; k0 += BATCH) {
    uint32_t hdr[BATCH][2], raw[BATCH][8];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int k = k0 + b;
#pragma unroll
      for (int i = 0; i < 8; ++i) raw[b][i] = 0;
      hdr[b][0] = hdr[b][1] = 0;
      if (ok[k] && k < live_rows) {
        if (RowTraits<TY>::quant) {
          hdr[b][0] = *reinterpret_cast<const uint32_t*>(row[k] + d.sb_off);
          if (d.sb_fp32) hdr[b][1] = *reinterpret_cast<const uint32_t*>(row[k] + d.sb_off + 4);
        }
        const uint8_t* p = row[k] + off;
        if constexpr (words == 8) {
          const Words4 a = *reinterpret_cast<const Words4*>(p), c = *reinterpret_cast<const Words4*>(p + 16);
#pragma unroll
          for (int i = 0; i < 4; ++i) { raw[b][i] = a.v[i]; raw[b][4 + i] = c.v[i]; }
        } else if constexpr (words == 4) {
          const Words4 a = *reinterpret_cast<const Words4*>(p);
#pragma unroll
          for (int i = 0; i < 4; ++i) raw[b][i] = a.v[i];
        } else if constexpr (words == 2) {
          const Words2 a = *reinterpret_cast<const Words2*>(p);
          raw[b][0] = a.v[0]; raw[b][1] = a.v[1];
        } else {
          raw[b][0] = *reinterpret_cast<const uint32_t*>(p);
        }
      }
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int k = k0 + b;
      if (k < live_rows) {
        float scale = 1.0f, bias = 0.0f;
        if (RowTraits<TY>::quant && ok[k]) {
          if (d.sb_fp32) {
            scale = 1.0f * s_bits_to_float(hdr[b][0]);
            bias = 1.0f * s_bits_to_float(hdr[b][1]);
          } else {
            scale = 1.0f * s_half_to_float((uint16_t)hdr[b][0]);
            bias = 1.0f * s_half_to_float((uint16_t)(hdr[b][0] >> 16));
          }
        }
        decode_store_t<TY>(raw[b], ok[k], 1.0f, scale, bias, j0, Dt, D, out_ty, orow0 + k * orow_step, fp8_shift, fp8_mult);
      }
    }
  }
}

__device__ __forceinline__ void emit_row(const TableDesc& d, const uint8_t* row, bool ok, float w, int D, int out_ty,
                                         uint8_t* orow, int sub, int lpr, int fp8_shift, float fp8_mult) {
  uint32_t hdr[2], raw[8];
  FBGEMM_AMD_ROW_TYPE_SWITCH(d.ty, (load_row_t<TY>(d, row, ok, D, sub, hdr, raw),
                                    finish_row_t<TY>(d, row, ok, w, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult, hdr, raw)))
}

template <typename index_t>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void sequence_lookup_kernel(
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
  const int64_t per_group = (int64_t)per_wave * SEQ_ROWS; // positions a wave takes per step
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t ngroups = (total_L + per_group - 1) / per_group;
  const bool copy_rows = out_ty == ST_INT8 || out_ty == ST_INT4;
  // bytes of an output row
  const int64_t out_row_bytes = out_ty == ST_FP32 ? (int64_t)D * 4 : (out_ty == ST_FP16 || out_ty == ST_BF16) ? (int64_t)D * 2
      : out_ty == ST_INT8 ? (int64_t)D + 4 : (int64_t)(D + 8 + 1) / 2;
  auto bound = [&](int t) -> int64_t { return in_lds ? bounds[t] : s_read(offsets, off64, (int64_t)t * B); };
  // the table of position `pos`: the largest t with bounds[t] <= pos (empty tables
  // share a boundary: the last of them wins)
  auto table_of = [&](int64_t pos) -> int {
    int lo = 0, hi = T; // invariant: bounds[lo] <= pos < bounds[hi] once the input is well formed
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (bound(mid) <= pos) lo = mid;
      else hi = mid;
    }
    return lo;
  };
  auto row_of = [&](const TableDesc& d, int64_t idx, int64_t pos, bool& ok) -> const uint8_t* {
    ok = true;
    if (idx == -1) {
      ok = false; // pruned row: zeros
    } else if (idx < 0 || idx >= d.num_rows) {
      if (sub == 0) {
        atomicOr(&status->bits, ERR_INDEX_OUT_OF_RANGE);
        atomicMin(&status->first_bad_pos, (unsigned long long)pos);
      }
      ok = false;
    }
    return (d.placement ? w1 : w0) + d.weights_offset + (ok ? idx : 0) * d.row_stride;
  };
  // A group of lpr lanes takes SEQ_ROWS positions per step, per_wave apart, so that
  // the wave's stores of one instruction still cover consecutive output rows. The
  // loads of all SEQ_ROWS rows are issued before the first is decoded; the indices
  // of the next step are fetched while they are in flight.
  int64_t g = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  int64_t idx[SEQ_ROWS];
#pragma unroll
  for (int k = 0; k < SEQ_ROWS; ++k) {
    const int64_t pos = g * per_group + (int64_t)k * per_wave + lane / lpr;
    idx[k] = (g < ngroups && pos < total_L) ? (int64_t)indices[pos] : 0;
  }
  while (g < ngroups) {
    const int64_t base = g * per_group + lane / lpr;
    const int64_t g2 = g + nwaves;
    int64_t idx2[SEQ_ROWS];
#pragma unroll
    for (int k = 0; k < SEQ_ROWS; ++k) {
      const int64_t pos2 = g2 * per_group + (int64_t)k * per_wave + lane / lpr;
      idx2[k] = (g2 < ngroups && pos2 < total_L) ? (int64_t)indices[pos2] : 0;
    }
    if (base < total_L) {
      // positions of one table (all but the steps that cross a table boundary) share its descriptor
      const int64_t last = base + (int64_t)(SEQ_ROWS - 1) * per_wave < total_L ? base + (int64_t)(SEQ_ROWS - 1) * per_wave : total_L - 1;
      const int t0 = table_of(base);
      const bool one_table = last < bound(t0 + 1);
      const int live_rows = (int)((last - base) / per_wave) + 1;
      TableDesc d = tables[t0];
      const uint8_t* row[SEQ_ROWS];
      bool ok[SEQ_ROWS];
      bool fast = one_table && !copy_rows && D <= lpr * SRUN;
      if (fast) {
        const int bits = s_type_bits(d.ty);
        const int run_bytes = (SRUN * bits) >> 3;
        const int b0 = (sub * SRUN * bits) >> 3;
        const int Dt = d.D < D ? d.D : D;
        fast = run_bytes >= 4 && b0 + run_bytes <= ((Dt * bits + 7) >> 3);
        uintptr_t misaligned = 0;
#pragma unroll
        for (int k = 0; k < SEQ_ROWS; ++k) {
          ok[k] = false;
          row[k] = nullptr;
          if (k < live_rows) {
            row[k] = row_of(d, idx[k], base + (int64_t)k * per_wave, ok[k]);
            misaligned |= reinterpret_cast<uintptr_t>(row[k] + d.sb_off) | reinterpret_cast<uintptr_t>(row[k] + d.data_off + b0);
          }
        }
        if (fast && (misaligned & 3) == 0) {
          FBGEMM_AMD_ROW_TYPE_SWITCH(d.ty, (rows_fast_t<TY>(d, row, ok, live_rows, D, out_ty,
                                                            reinterpret_cast<uint8_t*>(out) + base * out_row_bytes,
                                                            per_wave * out_row_bytes, sub, fp8_shift, fp8_mult)))
        } else {
          // this lane's run is partial, absent or off the dword grid: row by row (the checks are already made)
#pragma unroll 1
          for (int k = 0; k < live_rows; ++k)
            emit_row(d, row[k], ok[k], 1.0f, D, out_ty, reinterpret_cast<uint8_t*>(out) + (base + (int64_t)k * per_wave) * out_row_bytes,
                     sub, lpr, fp8_shift, fp8_mult);
        }
      } else {
#pragma unroll 1
        for (int k = 0; k < live_rows; ++k) {
          const int64_t pos = base + (int64_t)k * per_wave;
          if (!one_table) d = tables[table_of(pos)];
          uint8_t* orow = reinterpret_cast<uint8_t*>(out) + pos * out_row_bytes;
          bool okk;
          const uint8_t* r = row_of(d, idx[k], pos, okk);
          if (copy_rows) {
            // the row as it is stored: header, then elements (what fits the output row)
            const int64_t in_bytes = d.data_off + d.data_bytes;
            copy_row_bytes(r, okk, in_bytes < out_row_bytes ? in_bytes : out_row_bytes, out_row_bytes, orow, sub, lpr);
          } else {
            emit_row(d, r, okk, 1.0f, D, out_ty, orow, sub, lpr, fp8_shift, fp8_mult);
          }
        }
      }
    }
    g = g2;
#pragma unroll
    for (int k = 0; k < SEQ_ROWS; ++k) idx[k] = idx2[k];
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
  const int64_t per_block = 4 * (64 / lpr) * SEQ_ROWS;
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
