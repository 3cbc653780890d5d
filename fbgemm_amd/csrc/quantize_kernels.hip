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
// One wave per row; a lane owns runs of 8 consecutive elements.
#include <hip/hip_runtime.h>

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

// layout: 0 = data then (scale, bias) trailer; 1 = fp16 (scale, bias) header then data
template <bool HALF_IN>
__global__ __launch_bounds__(256) void quantize_rowwise_kernel(
    const void* input, int64_t rows, int32_t cols, int32_t bits, int32_t sb_float, int32_t layout,
    int64_t out_stride, uint8_t* output) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const void* in_row = reinterpret_cast<const uint8_t*>(input) + row * (int64_t)cols * (HALF_IN ? 2 : 4);
  uint8_t* out_row = output + row * out_stride;

  Extreme mn{0.0f, 0x7fffffff}, mx{0.0f, 0x7fffffff};
  for (int j0 = lane * RUN; j0 < cols; j0 += 64 * RUN) {
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
  for (int m = 1; m < 64; m <<= 1) {
    const Extreme on = shuffle_xor(mn, m), ox = shuffle_xor(mx, m);
    if (on.idx != 0x7fffffff) mn = mn.idx == 0x7fffffff ? on : first_min(mn, on);
    if (ox.idx != 0x7fffffff) mx = mx.idx == 0x7fffffff ? ox : first_max(mx, ox);
  }
  float minimum = mn.v;
  const float maximum = mx.v;

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
  if (lane == 0) {
    if (sb_bytes == 8) {
      for (int i = 0; i < 4; ++i) sb[i] = (uint8_t)(sb0 >> (8 * i));
      for (int i = 0; i < 4; ++i) sb[4 + i] = (uint8_t)(sb1 >> (8 * i));
    } else {
      sb[0] = (uint8_t)sb0; sb[1] = (uint8_t)(sb0 >> 8);
      sb[2] = (uint8_t)sb1; sb[3] = (uint8_t)(sb1 >> 8);
    }
  }
  for (int j0 = lane * RUN; j0 < cols; j0 += 64 * RUN) {
    uint32_t q[RUN];
    float xs[RUN];
    const int n = load_run<HALF_IN>(in_row, j0, cols, xs);
    for (int k = 0; k < RUN; ++k) {
      q[k] = 0;
      if (k < n) {
        const float x = xs[k];
        float r = __builtin_rintf((x - minimum) * inverse_scale); // lrintf: to nearest, ties to even
        if (clamp) r = r < 0.0f ? 0.0f : (r > (float)maxq ? (float)maxq : r);
        q[k] = (uint32_t)(int)r & 0xffu;
      }
    }
    // RUN elements = RUN * bits / 8 bytes, starting at a whole byte
    const int first_byte = j0 / epb;
    const int nbytes = RUN / epb;
    for (int b = 0; b < nbytes; ++b) {
      if (first_byte + b < data_bytes) {
        uint32_t byte = 0;
        for (int k = 0; k < epb; ++k) byte |= q[b * epb + k] << (k * bits);
        data[first_byte + b] = (uint8_t)byte;
      }
    }
  }
}

// output_ty: ST_FP32, ST_FP16, ST_BF16
__global__ __launch_bounds__(256) void dequantize_rowwise_kernel(
    const uint8_t* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t bits, int32_t sb_float,
    int32_t layout, int32_t output_ty, void* output) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint8_t* in_row = input + row * in_stride;
  const int epb = 8 / bits;
  const int data_bytes = (cols + epb - 1) / epb;
  const uint8_t* data = layout == 1 ? in_row + (sb_float ? 8 : 4) : in_row;
  const uint8_t* sb = layout == 1 ? in_row : in_row + data_bytes;
  float scale, bias;
  if (sb_float) {
    uint32_t u0 = 0, u1 = 0;
    for (int i = 0; i < 4; ++i) {
      u0 |= (uint32_t)sb[i] << (8 * i);
      u1 |= (uint32_t)sb[4 + i] << (8 * i);
    }
    scale = q_bits_to_float(u0);
    bias = q_bits_to_float(u1);
  } else {
    scale = half_bits_to_float((uint16_t)(sb[0] | (sb[1] << 8)));
    bias = half_bits_to_float((uint16_t)(sb[2] | (sb[3] << 8)));
  }
  const uint32_t mask = (1u << bits) - 1;
  for (int j = lane; j < cols; j += 64) {
    const uint32_t q = ((uint32_t)data[j / epb] >> ((j % epb) * bits)) & mask;
    const float v = (float)((double)scale * (double)q + (double)bias);
    const int64_t o = row * (int64_t)cols + j;
    if (output_ty == ST_FP32) reinterpret_cast<float*>(output)[o] = v;
    else if (output_ty == ST_FP16) reinterpret_cast<uint16_t*>(output)[o] = float_to_half_bits(v);
    else reinterpret_cast<uint16_t*>(output)[o] = float_to_bf16_bits(v);
  }
}

} // namespace

hipError_t launch_quantize_rowwise(const void* input, bool half_in, int64_t rows, int32_t cols, int32_t bits,
                                   int32_t sb_float, int32_t layout, int64_t out_stride, void* output,
                                   hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  if (half_in)
    hipLaunchKernelGGL(quantize_rowwise_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, input, rows, cols,
                       bits, sb_float, layout, out_stride, (uint8_t*)output);
  else
    hipLaunchKernelGGL(quantize_rowwise_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, input, rows, cols,
                       bits, sb_float, layout, out_stride, (uint8_t*)output);
  return hipGetLastError();
}

hipError_t launch_dequantize_rowwise(const void* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t bits,
                                     int32_t sb_float, int32_t layout, int32_t output_ty, void* output,
                                     hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(dequantize_rowwise_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)input,
                     rows, in_stride, cols, bits, sb_float, layout, output_ty, output);
  return hipGetLastError();
}

} // namespace fbgemm_amd
