// TEST INFRASTRUCTURE ONLY.
//
// C entry points over the reference's own scalar implementations, compiled
// from the reference's source files where they lie (see oracle/Makefile; the
// output goes to oracle/_ref/). The signatures mirror oracle/embedding_oracle.c
// one for one so that a test can call both with the same argument tuple and
// compare the bytes. No reference source is copied here: this file only
// includes the reference's headers and forwards to its templates
// (src/RefImplementations.h:221-330,408-453).
#include <cstdint>

#include "fbgemm/FloatConversion.h"
#include "src/RefImplementations.h"

namespace fbgemm {
// defined in src/RefImplementations.cc with external linkage
void Float8ToFloat_ref(const uint8_t input, float* output, int exponent_bits, int exponent_bias);
void FloatToFloat8_ref(const float input, uint8_t* output, int exponent_bits, int exponent_bias);
} // namespace fbgemm

namespace {

enum { ST_FP32 = 0, ST_FP16 = 1, ST_INT8 = 2, ST_INT4 = 3, ST_INT2 = 4, ST_BF16 = 5 };

struct Args {
  int in_ty;
  int64_t block_size, output_size, index_size, data_size;
  const void* input;
  const void* indices;
  const void* offsets;
  const float* weights;
  bool normalize;
  void* out;
  int out_ty;
  bool positional, use_offsets;
  int64_t output_stride, input_stride;
  bool scale_bias_last;
  const int32_t* remap;
};

template <typename I, typename O, typename Out>
bool run_typed(const Args& a) {
  const I* idx = static_cast<const I*>(a.indices);
  const O* off = static_cast<const O*>(a.offsets);
  Out* out = static_cast<Out*>(a.out);
  const bool bf16_out = a.out_ty == ST_BF16;
  if (a.remap) {
    // row-wise-sparse variants only produce float (RefImplementations.h:293-330)
    if constexpr (std::is_same_v<Out, float>) {
      switch (a.in_ty) {
        case ST_INT8:
          return fbgemm::EmbeddingSpMDMRowWiseSparse_ref<uint8_t, I, O>(
              a.block_size, a.output_size, a.index_size, a.data_size,
              static_cast<const uint8_t*>(a.input), idx, a.remap, off, a.weights,
              a.normalize, out, a.positional, a.use_offsets);
        case ST_INT4:
        case ST_INT2:
          return fbgemm::EmbeddingSpMDMNBitRowWiseSparse_ref<I, O>(
              a.in_ty == ST_INT4 ? 4 : 2, a.block_size, a.output_size, a.index_size,
              a.data_size, static_cast<const uint8_t*>(a.input), idx, a.remap, off,
              a.weights, a.normalize, out, a.positional, a.use_offsets);
        case ST_FP32:
          return fbgemm::EmbeddingSpMDMRowWiseSparse_ref<float, I, O>(
              a.block_size, a.output_size, a.index_size, a.data_size,
              static_cast<const float*>(a.input), idx, a.remap, off, a.weights,
              a.normalize, out, a.positional, a.use_offsets);
        case ST_FP16:
          return fbgemm::EmbeddingSpMDMRowWiseSparse_ref<uint16_t, I, O>(
              a.block_size, a.output_size, a.index_size, a.data_size,
              static_cast<const uint16_t*>(a.input), idx, a.remap, off, a.weights,
              a.normalize, out, a.positional, a.use_offsets);
        default:
          return false;
      }
    } else {
      return false;
    }
  }
  switch (a.in_ty) {
    case ST_INT8:
      return fbgemm::EmbeddingSpMDM_ref<uint8_t, I, O, Out>(
          a.block_size, a.output_size, a.index_size, a.data_size,
          static_cast<const uint8_t*>(a.input), idx, off, a.weights, a.normalize, out,
          a.positional, a.use_offsets, a.output_stride, a.input_stride,
          a.scale_bias_last, /*no_bag=*/false, bf16_out, false);
    case ST_INT4:
    case ST_INT2:
      return fbgemm::EmbeddingSpMDMNBit_ref<I, O, Out>(
          a.in_ty == ST_INT4 ? 4 : 2, a.block_size, a.output_size, a.index_size,
          a.data_size, static_cast<const uint8_t*>(a.input), idx, off, a.weights,
          a.normalize, out, a.positional, a.use_offsets, a.output_stride,
          a.input_stride, a.scale_bias_last, bf16_out, /*no_bag=*/false, -1);
    case ST_FP32:
      return fbgemm::EmbeddingSpMDM_ref<float, I, O, Out>(
          a.block_size, a.output_size, a.index_size, a.data_size,
          static_cast<const float*>(a.input), idx, off, a.weights, a.normalize, out,
          a.positional, a.use_offsets, a.output_stride, a.input_stride,
          a.scale_bias_last, false, bf16_out, false);
    case ST_FP16:
    case ST_BF16:
      return fbgemm::EmbeddingSpMDM_ref<uint16_t, I, O, Out>(
          a.block_size, a.output_size, a.index_size, a.data_size,
          static_cast<const uint16_t*>(a.input), idx, off, a.weights, a.normalize, out,
          a.positional, a.use_offsets, a.output_stride, a.input_stride,
          a.scale_bias_last, false, bf16_out, /*is_bf16_in=*/a.in_ty == ST_BF16);
    default:
      return false;
  }
}

template <typename I, typename O>
bool run_out(const Args& a) {
  if (a.out_ty == ST_FP32) return run_typed<I, O, float>(a);
  return run_typed<I, O, uint16_t>(a);
}

} // namespace

extern "C" {

int ref_embedding_spmdm(
    int in_ty, int64_t block_size, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* input, const void* indices, int idx64,
    const void* offsets_or_lengths, int off64, const float* weights,
    int normalize_by_lengths, void* out, int out_ty, int is_weight_positional,
    int use_offsets, int64_t output_stride, int64_t input_stride,
    int scale_bias_last, const int32_t* remap) {
  Args a{in_ty, block_size, output_size, index_size, data_size, input, indices,
         offsets_or_lengths, weights, normalize_by_lengths != 0, out, out_ty,
         is_weight_positional != 0, use_offsets != 0, output_stride, input_stride,
         scale_bias_last != 0, remap};
  bool ok;
  if (idx64) ok = off64 ? run_out<int64_t, int64_t>(a) : run_out<int64_t, int32_t>(a);
  else ok = off64 ? run_out<int32_t, int64_t>(a) : run_out<int32_t, int32_t>(a);
  return ok ? 1 : 0;
}

void ref_compressed_indices_remap(
    int32_t offsets_len, const void* indices, int idx64, const int32_t* mapping,
    const void* offsets, const float* weights, void* out_indices, void* out_offsets,
    float* out_weights) {
  if (idx64) {
    fbgemm::compressed_indices_remap_ref<int64_t>(
        offsets_len, static_cast<const int64_t*>(indices), mapping,
        static_cast<const int64_t*>(offsets), weights,
        static_cast<int64_t*>(out_indices), static_cast<int64_t*>(out_offsets),
        out_weights);
  } else {
    fbgemm::compressed_indices_remap_ref<int32_t>(
        offsets_len, static_cast<const int32_t*>(indices), mapping,
        static_cast<const int32_t*>(offsets), weights,
        static_cast<int32_t*>(out_indices), static_cast<int32_t*>(out_offsets),
        out_weights);
  }
}

float ref_float8_to_float(uint8_t input, int exponent_bits, int exponent_bias) {
  float f = 0.0f;
  fbgemm::Float8ToFloat_ref(input, &f, exponent_bits, exponent_bias);
  return f;
}

// EmbeddingSpMDMFP8_ref (src/RefImplementations.h:275-292); int64 indices and offsets, fp32 or 16-bit output
int ref_embedding_spmdm_fp8(
    int64_t block_size, int64_t output_size, int64_t index_size, int64_t data_size, const uint8_t* input,
    const int64_t* indices, const int64_t* offsets_or_lengths, const float* weights, int normalize_by_lengths,
    void* out, int out_ty, int is_weight_positional, int use_offsets, int64_t output_stride, int64_t input_stride,
    int exponent_bits, int exponent_bias) {
  if (out_ty == ST_FP32)
    return fbgemm::EmbeddingSpMDMFP8_ref<int64_t, int64_t, float>(
        block_size, output_size, index_size, data_size, input, indices, offsets_or_lengths, weights,
        normalize_by_lengths != 0, static_cast<float*>(out), is_weight_positional != 0, use_offsets != 0,
        output_stride, input_stride, exponent_bits, exponent_bias, false);
  return fbgemm::EmbeddingSpMDMFP8_ref<int64_t, int64_t, uint16_t>(
      block_size, output_size, index_size, data_size, input, indices, offsets_or_lengths, weights,
      normalize_by_lengths != 0, static_cast<uint16_t*>(out), is_weight_positional != 0, use_offsets != 0,
      output_stride, input_stride, exponent_bits, exponent_bias, out_ty == ST_BF16);
}

// The no_bag branches of EmbeddingSpMDM_ref / EmbeddingSpMDMNBit_ref (src/RefImplementations.cc:1235-1288,
// 1352-1376, 1466-1484); int64 indices. out_ty ST_INT8 / ST_INT4 select the byte-copy outputs.
int ref_embedding_spmdm_nobag(
    int in_ty, int64_t block_size, int64_t output_size, int64_t data_size, const void* input, const int64_t* indices,
    const float* weights, void* out, int out_ty, int64_t output_stride, int64_t input_stride, int scale_bias_last) {
  const bool sbl = scale_bias_last != 0;
  const bool bf16_out = out_ty == ST_BF16;
  const int32_t* no_offsets = nullptr;
#define NOBAG(IN, OUT, BF16IN)                                                                              \
  fbgemm::EmbeddingSpMDM_ref<IN, int64_t, int32_t, OUT>(                                                     \
      block_size, output_size, output_size, data_size, static_cast<const IN*>(input), indices, no_offsets, \
      weights, false, static_cast<OUT*>(out), false, true, output_stride, input_stride, sbl, /*no_bag=*/true, \
      bf16_out, BF16IN)
  switch (in_ty) {
    case ST_INT4:
    case ST_INT2:
      return fbgemm::EmbeddingSpMDMNBit_ref<int64_t, int32_t, uint8_t>(
          in_ty == ST_INT4 ? 4 : 2, block_size, output_size, output_size, data_size,
          static_cast<const uint8_t*>(input), indices, no_offsets, weights, false, static_cast<uint8_t*>(out), false,
          true, output_stride, input_stride, sbl, false, /*no_bag=*/true, out_ty == ST_INT4 ? 4 : -1);
    case ST_INT8:
      if (out_ty == ST_INT8) return NOBAG(uint8_t, uint8_t, false);
      if (out_ty == ST_FP32) return NOBAG(uint8_t, float, false);
      return NOBAG(uint8_t, uint16_t, false);
    case ST_FP32:
      if (out_ty == ST_FP32) return NOBAG(float, float, false);
      return NOBAG(float, uint16_t, false);
    case ST_FP16:
    case ST_BF16:
      if (out_ty == ST_FP32) return NOBAG(uint16_t, float, in_ty == ST_BF16);
      return NOBAG(uint16_t, uint16_t, in_ty == ST_BF16);
    default:
      return 0;
  }
#undef NOBAG
}

void ref_float_to_float8_array(const float* in, uint8_t* out, int64_t n, int exponent_bits, int exponent_bias) {
  for (int64_t i = 0; i < n; ++i) fbgemm::FloatToFloat8_ref(in[i], out + i, exponent_bits, exponent_bias);
}

float ref_half2float(uint16_t h) { return fbgemm::cpu_half2float(fbgemm::float16{h}); }
uint16_t ref_float2half_rn(float f) { return fbgemm::cpu_float2half_rn(f).val; }
uint16_t ref_float2bf16(float f) { return fbgemm::cpu_float2bfloat16(f).val; }

void ref_half2float_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = fbgemm::cpu_half2float(fbgemm::float16{in[i]});
}
void ref_float2half_rn_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = fbgemm::cpu_float2half_rn(in[i]).val;
}
void ref_float2bf16_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = fbgemm::cpu_float2bfloat16(in[i]).val;
}

} // extern "C"
