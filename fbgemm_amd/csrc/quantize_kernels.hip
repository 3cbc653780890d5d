// gfx950 kernels that produce and read the row-wise quantized formats the lookup
// consumes: fp32 / fp16 rows -> fused 8-, 4-, 2-bit rows with their scale and
// bias, and back.
//
// Arithmetic follows the reference's scalar code, operation for operation
// (src/QuantUtils.cc:534-611 N-bit with fp16 scale/bias, :677-718 8-bit with
// fp32 scale/bias, :743-789 and :847-892 the inverses):
//   N-bit: min rounded to fp16 (that is the stored bias); range = max - min;
//          scale = range == 0 ? 1 : range / (2^bits - 1), rounded to fp16, 1 if
//          that is 0 or its inverse overflows; q = clamp(lrintf((x - min) *
//          (1 / scale)), 0, 2^bits - 1); element j goes to bits
//          (j % epb) * bits of byte j / epb.
//   8-bit: scale = range / 255 and bias = min stored as fp32;
//          q = lrintf((x - min) * (255 / (range + 1e-8))).
//   back:  float(double(scale) * q + double(bias)), then one conversion.
// min / max are the FIRST smallest / largest element of the row, as
// std::min_element / std::max_element return them (this decides the sign of a
// zero bias or scale).
//
// `lpr` lanes (a power of two, chosen by the host from the row length) share a
// row and a lane owns runs of 8 consecutive elements, so a wave works on
// 64 / lpr rows at once: 16-byte loads, one store per run, and the row's
// elements stay in registers between the min/max pass and the rounding pass
// when one run per lane covers the row.
#include <hip/hip_runtime.h>

#include <cstring>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

__device__ __forceinline__ float q_bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t q_float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float half_bits_to_float(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t float_to_half_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); } // RNE
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) { return (uint16_t)((q_float_to_bits(f) + 0x8000u) >> 16); }

template <bool HALF_IN>
__device__ __forceinline__ float load_elem(const void* row, int64_t j) {
  if (HALF_IN) return half_bits_to_float(reinterpret_cast<const uint16_t*>(row)[j]);
  return reinterpret_cast<const float*>(row)[j];
}

constexpr int RUN = 8; // consecutive elements a lane handles at a time

// x[0..RUN) = elements j0 .. j0 + RUN of the row (those below cols); returns how many
template <bool HALF_IN>
__device__ __forceinline__ int load_run(const void* row, int j0, int cols, float (&x)[RUN]) {
  const uint8_t* p = reinterpret_cast<const uint8_t*>(row) + (int64_t)j0 * (HALF_IN ? 2 : 4);
  if (j0 + RUN <= cols && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    if (HALF_IN) {
      const uint4 v = *reinterpret_cast<const uint4*>(p);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      for (int k = 0; k < 4; ++k) {
        x[2 * k] = half_bits_to_float((uint16_t)w[k]);
        x[2 * k + 1] = half_bits_to_float((uint16_t)(w[k] >> 16));
      }
    } else {
      const float4 a = reinterpret_cast<const float4*>(p)[0];
      const float4 b = reinterpret_cast<const float4*>(p)[1];
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
      x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
    return RUN;
  }
  int n = 0;
  for (int k = 0; k < RUN; ++k) {
    x[k] = 0.0f;
    if (j0 + k < cols) {
      x[k] = load_elem<HALF_IN>(row, j0 + k);
      n = k + 1;
    }
  }
  return n;
}

struct Extreme {
  float v;
  int idx;
};
// first smallest: smaller value wins, equal values (+0 / -0 included) keep the lower index
__device__ __forceinline__ Extreme first_min(Extreme a, Extreme b) {
  if (b.v < a.v || (!(a.v < b.v) && b.idx < a.idx)) return b;
  return a;
}
__device__ __forceinline__ Extreme first_max(Extreme a, Extreme b) {
  if (a.v < b.v || (!(b.v < a.v) && b.idx < a.idx)) return b;
  return a;
}
__device__ __forceinline__ Extreme shuffle_xor(Extreme e, int mask) {
  Extreme r;
  r.v = __shfl_xor(e.v, mask, 64);
  r.idx = __shfl_xor(e.idx, mask, 64);
  return r;
}

// stores the nbytes (1, 2, 4 or 8) of one run of quantized elements
__device__ __forceinline__ void store_run(uint8_t* p, uint64_t v, int nbytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  if (nbytes == 8 && (a & 3) == 0) {
    reinterpret_cast<uint32_t*>(p)[0] = (uint32_t)v;
    reinterpret_cast<uint32_t*>(p)[1] = (uint32_t)(v >> 32);
  } else if (nbytes == 4 && (a & 3) == 0) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)v;
  } else if (nbytes == 2 && (a & 1) == 0) {
    *reinterpret_cast<uint16_t*>(p) = (uint16_t)v;
  } else {
    for (int b = 0; b < nbytes; ++b) p[b] = (uint8_t)(v >> (8 * b));
  }
}

// layout: 0 = data then (scale, bias) trailer; 1 = fp16 (scale, bias) header then data
template <bool HALF_IN, int BITS>
__global__ __launch_bounds__(256) void quantize_rowwise_kernel(
    const void* input, int64_t rows, int32_t cols_arg, int32_t sb_float, int32_t layout,
    int64_t out_stride, uint8_t* output, int32_t lpr, const int32_t* seg_offsets, int32_t seg_T, int64_t seg_in_stride,
    const void* min_max, const int32_t* seg_tables) {
  constexpr int bits = BITS;
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int rows_per_wave = 64 / lpr;
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t ngroups = (rows + rows_per_wave - 1) / rows_per_wave;
  // every wave walks row groups wave, wave + nwaves, ...: the loop bound is the same for all lanes of a wave
  for (int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); wave < ngroups; wave += nwaves) {
  const int64_t row_raw = wave * rows_per_wave + lane / lpr;
  const bool live = row_raw < rows;
  const int64_t row = live ? row_raw : rows - 1; // lanes past the end shadow the last row and store nothing
  // Segment mode (seg_offsets != null): "row" r is the segment of table t = r % seg_T in
  // line b = r / seg_T of a [lines, seg_in_stride] matrix: columns seg_offsets[t] .. seg_offsets[t+1],
  // quantized to seg_offsets[t] + t * 8 bytes into line b of the output (every segment carries its
  // own 8 bytes of scale and bias behind its data). With seg_tables the segments are those of the
  // seg_T tables it lists (t = seg_tables[r % seg_T]) and the others are left alone.
  int32_t cols = cols_arg;
  const void* in_row;
  uint8_t* out_row;
  if (seg_offsets) {
    const int64_t b = row / seg_T;
    int32_t t = (int32_t)(row - b * seg_T);
    if (seg_tables) t = seg_tables[t];
    const int32_t c0 = seg_offsets[t];
    cols = seg_offsets[t + 1] - c0;
    in_row = reinterpret_cast<const uint8_t*>(input) + (b * seg_in_stride + c0) * (HALF_IN ? 2 : 4);
    out_row = output + b * out_stride + c0 + (int64_t)t * 8;
  } else {
    in_row = reinterpret_cast<const uint8_t*>(input) + row * (int64_t)cols * (HALF_IN ? 2 : 4);
    out_row = output + row * out_stride;
  }
  const bool single = cols <= lpr * RUN; // one run per lane covers the row

  // Fast pass: plain minimum / maximum. Which of several equal extremes is
  // taken only shows when the extreme is a zero and zeros of both signs are in
  // the row (the sign of the stored bias / of max - min); a wave that meets a
  // zero extreme redoes the search with positions (the first extreme wins, as
  // std::min_element / std::max_element choose).
  float lo = __builtin_inff(), hi = -__builtin_inff();
  float keep[RUN];
  int keep_n = 0;
  for (int j0 = sub * RUN; j0 < cols; j0 += lpr * RUN) {
    float x[RUN];
    const int n = load_run<HALF_IN>(in_row, j0, cols, x);
    for (int k = 0; k < RUN; ++k) {
      keep[k] = x[k];
      if (k < n) {
        lo = x[k] < lo ? x[k] : lo;
        hi = hi < x[k] ? x[k] : hi;
      }
    }
    keep_n = n;
  }
  for (int m = 1; m < lpr; m <<= 1) {
    const float ol = __shfl_xor(lo, m, 64), oh = __shfl_xor(hi, m, 64);
    lo = ol < lo ? ol : lo;
    hi = hi < oh ? oh : hi;
  }
  Extreme mn{lo, 0}, mx{hi, 0};
  if (__builtin_amdgcn_ballot_w64(lo == 0.0f || hi == 0.0f) != 0ull) {
    mn = Extreme{0.0f, 0x7fffffff};
    mx = Extreme{0.0f, 0x7fffffff};
    for (int j0 = sub * RUN; j0 < cols; j0 += lpr * RUN) {
      float x[RUN];
      const int n = load_run<HALF_IN>(in_row, j0, cols, x);
      for (int k = 0; k < RUN; ++k) {
        if (k < n) {
          const Extreme e{x[k], j0 + k};
          mn = mn.idx == 0x7fffffff ? e : first_min(mn, e);
          mx = mx.idx == 0x7fffffff ? e : first_max(mx, e);
        }
      }
    }
    for (int m = 1; m < lpr; m <<= 1) {
      const Extreme on = shuffle_xor(mn, m), ox = shuffle_xor(mx, m);
      if (on.idx != 0x7fffffff) mn = mn.idx == 0x7fffffff ? on : first_min(mn, on);
      if (ox.idx != 0x7fffffff) mx = mx.idx == 0x7fffffff ? ox : first_max(mx, ox);
    }
  }
  float minimum = mn.v;
  float maximum = mx.v;
  // Extremes the caller brings (two input-typed values per row, minimum then maximum) take the
  // place of the ones found (src/QuantUtilsAvx2.cc:1605-1628, :1831-1853).
  if (min_max) {
    if (HALF_IN) {
      const uint16_t* mm = reinterpret_cast<const uint16_t*>(min_max) + row * 2;
      minimum = half_bits_to_float(mm[0]);
      maximum = half_bits_to_float(mm[1]);
    } else {
      const float* mm = reinterpret_cast<const float*>(min_max) + row * 2;
      minimum = mm[0];
      maximum = mm[1];
    }
  }

  const int epb = 8 / bits;
  const int data_bytes = (cols + epb - 1) / epb;
  const int maxq = (1 << bits) - 1;
  float inverse_scale;
  uint32_t sb0, sb1; // what is stored: bit patterns of scale and bias
  bool clamp;
  if (sb_float) {
    // QuantUtils.cc:704-715
    const float range = maximum - minimum;
    sb0 = q_float_to_bits(range / 255.0f);
    sb1 = q_float_to_bits(minimum);
    inverse_scale = 255.0f / (range + 1e-8f);
    clamp = false;
  } else {
    // QuantUtils.cc:573-596
    const uint16_t min16 = float_to_half_bits(minimum);
    minimum = half_bits_to_float(min16);
    const float range = maximum - minimum;
    float scale = range == 0.0f ? 1.0f : range / (float)maxq;
    scale = half_bits_to_float(float_to_half_bits(scale));
    if (scale == 0.0f) scale = 1.0f;
    inverse_scale = 1.0f / scale;
    if (__builtin_isinf(inverse_scale)) {
      scale = 1.0f;
      inverse_scale = 1.0f;
    }
    sb0 = float_to_half_bits(scale);
    sb1 = min16;
    clamp = true;
  }
  // TBE rows carry an fp16 pair in front whatever the source format stored
  // (fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:47-70)
  int sb_bytes = sb_float ? 8 : 4;
  if (layout == 1 && sb_float) {
    sb0 = float_to_half_bits(q_bits_to_float(sb0));
    sb1 = float_to_half_bits(q_bits_to_float(sb1));
    sb_bytes = 4;
  }
  uint8_t* data = layout == 1 ? out_row + 4 : out_row;
  uint8_t* sb = layout == 1 ? out_row : out_row + data_bytes;
  if (live && sub == 0) {
    if (sb_bytes == 8) store_run(sb, (uint64_t)sb0 | ((uint64_t)sb1 << 32), 8);
    else store_run(sb, (uint64_t)(sb0 & 0xffffu) | ((uint64_t)(sb1 & 0xffffu) << 16), 4);
  }
  const int run_bytes = RUN / epb;
  const int wrap_from = cols & ~31;
  for (int j0 = sub * RUN; j0 < cols; j0 += lpr * RUN) {
    float xs[RUN];
    int n;
    if (single) {
      for (int k = 0; k < RUN; ++k) xs[k] = keep[k];
      n = keep_n;
    } else {
      n = load_run<HALF_IN>(in_row, j0, cols, xs);
    }
    uint32_t w0 = 0, w1 = 0; // the run's bytes: RUN * bits <= 32 bits fill w0; 8-bit runs use both
    for (int k = 0; k < RUN; ++k) {
      if (k < n) {
        float r = __builtin_rintf((xs[k] - minimum) * inverse_scale); // lrintf: to nearest, ties to even
        // Only elements outside extremes that the caller brought can leave 0 .. maxq in the 8-bit
        // float-pair format. The reference's vector code then saturates the leading whole groups
        // of 32 columns and keeps the low byte of the rounded integer in the columns behind them;
        // a value that does not fit 32 bits converts to 0x80000000 there, which both rules turn
        // into 0 (src/QuantUtilsAvx2.cc:1912-1950).
        if (clamp) {
          // fp16-pair formats clamp the rounded value as a 32-bit integer. Beyond 32 bits (extremes
          // from the caller only) that integer is 0x80000000 in the whole groups of 32 columns of
          // the 2- and 4-bit formats and the low half of the 64-bit integer in the other columns
          // (src/QuantUtilsAvx2.cc:1697-1722, :1768-1773).
          if (min_max && !(__builtin_fabsf(r) < 2147483648.0f)) {
            if ((bits < 8 && j0 + k < wrap_from) || !(__builtin_fabsf(r) < 9223372036854775808.0f)) r = 0.0f;
            else r = (float)(int32_t)(uint32_t)(uint64_t)(int64_t)r;
          }
          r = r < 0.0f ? 0.0f : (r > (float)maxq ? (float)maxq : r);
        } else if (min_max) {
          if (!(__builtin_fabsf(r) < 2147483648.0f)) r = 0.0f;
          else if (j0 + k < wrap_from) r = r < 0.0f ? 0.0f : (r > 255.0f ? 255.0f : r);
        }
        const uint32_t q = (uint32_t)(int)r & 0xffu;
        if (bits == 8 && k >= 4) w1 |= q << ((k - 4) * 8);
        else w0 |= q << (k * bits);
      }
    }
    const uint64_t packed = (uint64_t)w0 | ((uint64_t)w1 << 32);
    // RUN elements = RUN * bits / 8 bytes, starting at a whole byte
    const int first_byte = j0 / epb;
    const int nb = data_bytes - first_byte < run_bytes ? data_bytes - first_byte : run_bytes;
    if (live) store_run(data + first_byte, packed, nb);
  }
  }
}

// output_ty: ST_FP32, ST_FP16, ST_BF16. `lpr` lanes share a row; a lane turns
// runs of 4 packed elements into 4 outputs (one 16-byte store of fp32: every
// store instruction of the wave then writes whole contiguous lines).
constexpr int DRUN = 4;
template <int BITS>
__global__ __launch_bounds__(256) void dequantize_rowwise_kernel(
    const uint8_t* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t sb_float,
    int32_t layout, int32_t output_ty, void* output, int32_t lpr) {
  constexpr int bits = BITS;
  const int lane = threadIdx.x & 63;
  const int sub = lane & (lpr - 1);
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
  for (int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);; wave += nwaves) {
  const int64_t row = wave * (64 / lpr) + lane / lpr;
  if (row >= rows) return;
  const uint8_t* in_row = input + row * in_stride;
  const int epb = 8 / bits;
  const int data_bytes = (cols + epb - 1) / epb;
  const uint8_t* data = layout == 1 ? in_row + (sb_float ? 8 : 4) : in_row;
  const uint8_t* sb = layout == 1 ? in_row : in_row + data_bytes;
  float scale, bias;
  if (sb_float) {
    uint32_t u0 = 0, u1 = 0;
    if ((reinterpret_cast<uintptr_t>(sb) & 3) == 0) {
      u0 = reinterpret_cast<const uint32_t*>(sb)[0];
      u1 = reinterpret_cast<const uint32_t*>(sb)[1];
    } else {
      for (int i = 0; i < 4; ++i) {
        u0 |= (uint32_t)sb[i] << (8 * i);
        u1 |= (uint32_t)sb[4 + i] << (8 * i);
      }
    }
    scale = q_bits_to_float(u0);
    bias = q_bits_to_float(u1);
  } else {
    uint32_t u;
    if ((reinterpret_cast<uintptr_t>(sb) & 3) == 0) u = *reinterpret_cast<const uint32_t*>(sb);
    else u = sb[0] | (sb[1] << 8) | (sb[2] << 16) | ((uint32_t)sb[3] << 24);
    scale = half_bits_to_float((uint16_t)u);
    bias = half_bits_to_float((uint16_t)(u >> 16));
  }
  const uint32_t mask = (1u << bits) - 1;
  const int run_bytes = DRUN / epb; // 4, 2 or 1
  for (int j0 = sub * DRUN; j0 < cols; j0 += lpr * DRUN) {
    const uint8_t* p = data + j0 / epb;
    const int nb = data_bytes - j0 / epb < run_bytes ? data_bytes - j0 / epb : run_bytes;
    uint32_t packed = 0;
    const uintptr_t pa = reinterpret_cast<uintptr_t>(p);
    if (nb == 4 && (pa & 3) == 0) packed = *reinterpret_cast<const uint32_t*>(p);
    else if (nb == 2 && (pa & 1) == 0) packed = *reinterpret_cast<const uint16_t*>(p);
    else for (int b = 0; b < nb; ++b) packed |= (uint32_t)p[b] << (8 * b);
    float v[DRUN];
    for (int k = 0; k < DRUN; ++k) {
      const uint32_t q = (packed >> (k * bits)) & mask;
      v[k] = (float)((double)scale * (double)q + (double)bias);
    }
    const int n = cols - j0 < DRUN ? cols - j0 : DRUN;
    const int64_t o = row * (int64_t)cols + j0;
    if (output_ty == ST_FP32) {
      float* op = reinterpret_cast<float*>(output) + o;
      if (n == DRUN && (reinterpret_cast<uintptr_t>(op) & 15) == 0) {
        stream_store16(op, v[0], v[1], v[2], v[3]);
      } else {
        for (int k = 0; k < DRUN; ++k) if (k < n) op[k] = v[k];
      }
    } else {
      uint16_t h[DRUN];
      for (int k = 0; k < DRUN; ++k) h[k] = output_ty == ST_FP16 ? float_to_half_bits(v[k]) : float_to_bf16_bits(v[k]);
      uint16_t* op = reinterpret_cast<uint16_t*>(output) + o;
      if (n == DRUN && (reinterpret_cast<uintptr_t>(op) & 7) == 0) {
        stream_store8(op, h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
      } else {
        for (int k = 0; k < DRUN; ++k) if (k < n) op[k] = h[k];
      }
    }
  }
  }
}

// fp32 -> 8-bit float (hfp8), the reference's float_to_hfp8
// (fbgemm_gpu/include/fbgemm_gpu/quantize_ops_utils.h:29-81; the same steps as
// FloatToFloat8_ref, src/RefImplementations.cc:126-182): |x| clamped to max_pos;
// in the normal range a power of two 23 - mbits binades above x is added and
// subtracted, so that fp32's round-to-nearest-even rounds x to mbits mantissa
// bits; below the smallest normal 2^(24 - bias - mbits) is added and the low
// bits of the sum are the code. The sign goes to bit 7.
__device__ __forceinline__ uint32_t float_to_hfp8(float x, int ebits, int bias, float max_pos) {
  const int mbits = 7 - ebits;
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  const uint32_t sign = u & 0x80000000u;
  u &= 0x7fffffffu;
  const float v = __builtin_fminf(__builtin_bit_cast(float, u), max_pos);
  u = __builtin_bit_cast(uint32_t, v);
  const float smallest_normal = __builtin_bit_cast(float, (uint32_t)(127 - bias + 1) << 23);
  if (v >= smallest_normal) {
    const float bouncer = __builtin_bit_cast(float, (u & 0xff800000u) + ((uint32_t)(23 - mbits) << 23));
    const float r = (bouncer + v) - bouncer;
    uint32_t o = (__builtin_bit_cast(uint32_t, r) - ((uint32_t)(127 - bias) << 23)) << (8 - ebits);
    return ((o | sign) >> 24) & 0xffu;
  }
  const float bouncer = __builtin_bit_cast(float, (uint32_t)(127 + (23 + (1 - bias - mbits))) << 23);
  const float r = bouncer + v;
  return (__builtin_bit_cast(uint32_t, r) | (sign >> 24)) & 0xffu;
}

// hfp8 -> fp32 (hfp8_to_float, quantize_ops_utils.h:83-110; Float8ToFloat_ref)
__device__ __forceinline__ float hfp8_to_float(uint32_t b, int shift, float mult) {
  const float mag = __builtin_bit_cast(float, (b & 0x7fu) << shift) * mult;
  return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, mag) | ((b & 0x80u) << 24));
}

// Four elements per lane and step: one 16-byte load or store on the fp32 side,
// one 4-byte access on the code side; the tail (and unaligned buffers) element by element.
__global__ __launch_bounds__(256) void float_to_hfp8_kernel(const float* in, uint8_t* out, int64_t n, int ebits,
                                                            int bias, float max_pos) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const bool vec = (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 3) == 0;
  const int64_t n4 = vec ? n / 4 : 0;
  for (int64_t i = tid; i < n4; i += nthreads) {
    const float4 x = reinterpret_cast<const float4*>(in)[i];
    const uint32_t c = float_to_hfp8(x.x, ebits, bias, max_pos) | (float_to_hfp8(x.y, ebits, bias, max_pos) << 8) |
        (float_to_hfp8(x.z, ebits, bias, max_pos) << 16) | (float_to_hfp8(x.w, ebits, bias, max_pos) << 24);
    stream_store4(reinterpret_cast<uint32_t*>(out) + i, c);
  }
  for (int64_t i = n4 * 4 + tid; i < n; i += nthreads) out[i] = (uint8_t)float_to_hfp8(in[i], ebits, bias, max_pos);
}

__global__ __launch_bounds__(256) void hfp8_to_float_kernel(const uint8_t* in, float* out, int64_t n, int shift, float mult) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const bool vec = (reinterpret_cast<uintptr_t>(in) & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const int64_t n4 = vec ? n / 4 : 0;
  for (int64_t i = tid; i < n4; i += nthreads) {
    const uint32_t c = reinterpret_cast<const uint32_t*>(in)[i];
    stream_store16(reinterpret_cast<float4*>(out) + i, hfp8_to_float(c & 0xffu, shift, mult), hfp8_to_float((c >> 8) & 0xffu, shift, mult),
                   hfp8_to_float((c >> 16) & 0xffu, shift, mult), hfp8_to_float(c >> 24, shift, mult));
  }
  for (int64_t i = n4 * 4 + tid; i < n; i += nthreads) out[i] = hfp8_to_float(in[i], shift, mult);
}

// enough workgroups to fill the device several times over, no more than there is work
unsigned stream_blocks(int64_t needed) {
  const int64_t cap = 256 * 64;
  return (unsigned)(needed < cap ? (needed < 1 ? 1 : needed) : cap);
}

// lanes per row: the power of two (1..64) that gives a lane about one run
int lanes_per_row(int32_t cols, int run) {
  int lpr = 1;
  while (lpr < 64 && lpr * run < cols) lpr <<= 1;
  return lpr;
}

} // namespace

hipError_t launch_quantize_rowwise(const void* input, bool half_in, int64_t rows, int32_t cols, int32_t bits,
                                   int32_t sb_float, int32_t layout, int64_t out_stride, void* output,
                                   const void* min_max, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  const int lpr = lanes_per_row(cols, RUN);
  const int64_t rows_per_block = 4 * (64 / lpr);
  const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  const dim3 grid(stream_blocks(blocks)), block(256);
#define FBGEMM_AMD_LAUNCH_Q(H, B) \
  hipLaunchKernelGGL((quantize_rowwise_kernel<H, B>), grid, block, 0, stream, input, rows, cols, sb_float, layout, \
                     out_stride, (uint8_t*)output, lpr, (const int32_t*)nullptr, 0, (int64_t)0, min_max, (const int32_t*)nullptr)
  if (half_in) {
    if (bits == 2) FBGEMM_AMD_LAUNCH_Q(true, 2);
    else if (bits == 4) FBGEMM_AMD_LAUNCH_Q(true, 4);
    else FBGEMM_AMD_LAUNCH_Q(true, 8);
  } else {
    if (bits == 2) FBGEMM_AMD_LAUNCH_Q(false, 2);
    else if (bits == 4) FBGEMM_AMD_LAUNCH_Q(false, 4);
    else FBGEMM_AMD_LAUNCH_Q(false, 8);
  }
#undef FBGEMM_AMD_LAUNCH_Q
  return hipGetLastError();
}

// Every (line, table) segment of a [lines, total_D] fp32 matrix to 8-bit rows with an fp32
// (scale, bias) trailer each: line b of the output holds, for t = 0 .. T-1, D_t bytes and 8 bytes.
// d_tables (or null): the n_tables tables whose segments are quantized; the others are left alone.
hipError_t launch_quantize_segments(const float* input, int64_t lines, int32_t T, const int32_t* d_seg_offsets,
                                    int32_t total_D, int32_t max_D, uint8_t* output, const int32_t* d_tables,
                                    int32_t n_tables, hipStream_t stream) {
  if (lines <= 0 || T <= 0 || max_D <= 0 || (d_tables && n_tables <= 0)) return hipSuccess;
  const int lpr = lanes_per_row(max_D, RUN);
  const int32_t seg_T = d_tables ? n_tables : T;
  const int64_t rows = lines * seg_T;
  const int64_t rows_per_block = 4 * (64 / lpr);
  const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  const dim3 grid(stream_blocks(blocks)), block(256);
  hipLaunchKernelGGL((quantize_rowwise_kernel<false, 8>), grid, block, 0, stream, (const void*)input, rows, max_D, 1, 0,
                     (int64_t)total_D + 8 * (int64_t)T, output, lpr, d_seg_offsets, seg_T, (int64_t)total_D,
                     (const void*)nullptr, d_tables);
  return hipGetLastError();
}

hipError_t launch_dequantize_rowwise(const void* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t bits,
                                     int32_t sb_float, int32_t layout, int32_t output_ty, void* output,
                                     hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  const int lpr = lanes_per_row(cols, DRUN);
  const int64_t rows_per_block = 4 * (64 / lpr);
  const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  const dim3 grid(stream_blocks(blocks)), block(256);
#define FBGEMM_AMD_LAUNCH_D(B) \
  hipLaunchKernelGGL((dequantize_rowwise_kernel<B>), grid, block, 0, stream, (const uint8_t*)input, rows, in_stride, \
                     cols, sb_float, layout, output_ty, output, lpr)
  if (bits == 2) FBGEMM_AMD_LAUNCH_D(2);
  else if (bits == 4) FBGEMM_AMD_LAUNCH_D(4);
  else FBGEMM_AMD_LAUNCH_D(8);
#undef FBGEMM_AMD_LAUNCH_D
  return hipGetLastError();
}

hipError_t launch_float_to_hfp8(const float* input, int64_t n, int32_t ebits, int32_t bias, float max_pos, uint8_t* output,
                                hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const dim3 grid(stream_blocks((n / 4 + 255) / 256)), block(256);
  hipLaunchKernelGGL(float_to_hfp8_kernel, grid, block, 0, stream, input, output, n, ebits, bias, max_pos);
  return hipGetLastError();
}

hipError_t launch_hfp8_to_float(const uint8_t* input, int64_t n, int32_t ebits, int32_t bias, float* output, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const uint32_t mult_bits = (uint32_t)(127 + (127 - bias)) << 23; // 2^(127 - bias)
  float mult;
  memcpy(&mult, &mult_bits, 4);
  const dim3 grid(stream_blocks((n / 4 + 255) / 256)), block(256);
  hipLaunchKernelGGL(hfp8_to_float_kernel, grid, block, 0, stream, input, output, n, 16 + ebits, mult);
  return hipGetLastError();
}

} // namespace fbgemm_amd
