// C++ face of the C ABI, shaped like include/fbgemm/FbgemmEmbedding.h of the
// reference: the same factory templates with the same argument lists, returning
// std::function objects with the EmbeddingSpMDMKernelSignature call signature.
//
// Differences a caller must know:
//   * every pointer passed to a generated kernel is a DEVICE pointer;
//   * the kernel runs on the stream set with fbgemm_amd::set_stream() (default
//     stream otherwise) and, like the reference, returns only when done, with
//     the reference's bool;
//   * `prefetch` and THREAD_LOCAL are accepted and ignored (they tune the CPU
//     code generator). Kernels may be called from several host threads at once,
//     as the reference's may: every thread has its own stream setting, status
//     block and scratch buffers inside the library. Calls of one thread run one
//     after the other (each returns when its work is done);
// Header-only; link against libfbgemm_amd.so.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "fbgemm_amd.h"

namespace fbgemm_amd {

// 16-bit storage types, as in the reference's include/fbgemm/Types.h.
struct float16 { std::uint16_t val; };
struct bfloat16 { std::uint16_t val; };

inline void*& stream_ref() {
  static thread_local void* s = nullptr;
  return s;
}
// Stream (hipStream_t) the kernels generated on this thread run on.
inline void set_stream(void* hip_stream) { stream_ref() = hip_stream; }

template <typename InType, typename IndexType, typename OffsetType = std::int32_t, typename OutType = float>
class EmbeddingSpMDMKernelSignature {
 public:
  using Type = std::function<bool(
      std::int64_t output_size, std::int64_t index_size, std::int64_t data_size, const InType* input,
      const IndexType* indices, const OffsetType* offsets_or_lengths,
      const float* weights, // optional, can be null for non-weighted sum
      OutType* out)>;
};

template <typename InType, typename IndexType, typename OffsetType = std::int32_t>
class EmbeddingSpMDMRowWiseSparseKernelSignature {
 public:
  using Type = std::function<bool(
      std::int64_t output_size, std::int64_t index_size, std::int64_t uncompressed_data_size,
      const InType* input, const IndexType* indices, const OffsetType* offsets_or_lengths,
      const float* weights, float* out, const std::int32_t* compressed_indices_table)>;
};

namespace detail {

template <typename T>
constexpr int bits_of() {
  static_assert(std::is_same_v<T, std::int32_t> || std::is_same_v<T, std::int64_t>, "index/offset type must be int32 or int64");
  return sizeof(T) * 8;
}

template <typename InType>
constexpr int weight_ty(bool is_bf16_in) {
  if constexpr (std::is_same_v<InType, std::uint8_t>) return FBGEMM_AMD_INT8;
  else if constexpr (std::is_same_v<InType, float>) return FBGEMM_AMD_FP32;
  else if constexpr (std::is_same_v<InType, float16> || std::is_same_v<InType, std::uint16_t>)
    return is_bf16_in ? FBGEMM_AMD_BF16 : FBGEMM_AMD_FP16;
  else static_assert(sizeof(InType) == 0, "InType must be uint8_t, float16, uint16_t or float");
}

template <typename OutType>
constexpr int output_ty(bool is_bf16_out) {
  if constexpr (std::is_same_v<OutType, float>) return FBGEMM_AMD_FP32;
  else if constexpr (std::is_same_v<OutType, float16> || std::is_same_v<OutType, std::uint16_t>)
    return is_bf16_out ? FBGEMM_AMD_BF16 : FBGEMM_AMD_FP16;
  else if constexpr (std::is_same_v<OutType, bfloat16>) return FBGEMM_AMD_BF16;
  // rows copied as stored (no_bag only): the C ABI rejects this type for the pooled kernels
  else if constexpr (std::is_same_v<OutType, std::uint8_t>) return FBGEMM_AMD_INT8;
  else static_assert(sizeof(OutType) == 0, "OutType must be float, float16, uint16_t, bfloat16 or (no_bag) uint8_t");
}

inline bool run(const fbgemm_amd_spmdm_config& cfg, std::int64_t output_size, std::int64_t index_size,
                std::int64_t data_size, const void* input, const void* indices, const void* offsets,
                const float* weights, void* out, const std::int32_t* table, bool has_weight) {
  if (has_weight != (weights != nullptr))
    throw std::invalid_argument("fbgemm_amd: weights must be given exactly when has_weight was set");
  const int rc = fbgemm_amd_spmdm_run(&cfg, output_size, index_size, data_size, input, indices, offsets, weights,
                                      out, table, stream_ref());
  if (rc < 0) throw std::runtime_error(std::string("fbgemm_amd: ") + fbgemm_amd_last_error());
  return rc == 1;
}

} // namespace detail

// GenerateEmbeddingSpMDMWithStrides (FbgemmEmbedding.h:94-117)
template <typename InType, typename IndexType, typename OffsetType = std::int32_t, typename OutType = float,
          bool THREAD_LOCAL = false>
typename EmbeddingSpMDMKernelSignature<InType, IndexType, OffsetType, OutType>::Type
GenerateEmbeddingSpMDMWithStrides(const std::int64_t block_size, bool has_weight, bool normalize_by_lengths,
                                  int /*prefetch*/ = 16, bool is_weight_positional = false, bool use_offsets = true,
                                  std::int64_t output_stride = -1, std::int64_t input_stride = -1,
                                  bool scale_bias_last = true, bool no_bag = false, bool is_bf16_out = false,
                                  bool is_bf16_in = false) {
  fbgemm_amd_spmdm_config cfg{};
  cfg.no_bag = no_bag;
  cfg.weight_ty = detail::weight_ty<InType>(is_bf16_in);
  cfg.output_ty = detail::output_ty<OutType>(is_bf16_out);
  cfg.index_bits = detail::bits_of<IndexType>();
  cfg.offset_bits = detail::bits_of<OffsetType>();
  cfg.block_size = block_size;
  cfg.output_stride = output_stride;
  cfg.input_stride = input_stride;
  cfg.normalize_by_lengths = normalize_by_lengths;
  cfg.is_weight_positional = is_weight_positional;
  cfg.use_offsets = use_offsets;
  cfg.scale_bias_last = scale_bias_last;
  return [cfg, has_weight](std::int64_t output_size, std::int64_t index_size, std::int64_t data_size,
                           const InType* input, const IndexType* indices, const OffsetType* offsets_or_lengths,
                           const float* weights, OutType* out) {
    return detail::run(cfg, output_size, index_size, data_size, input, indices, offsets_or_lengths, weights, out,
                       nullptr, has_weight);
  };
}

// GenerateEmbeddingSpMDM (FbgemmEmbedding.h:65-84)
template <typename InType, typename IndexType, typename OffsetType = std::int32_t, typename OutType = float,
          bool THREAD_LOCAL = false>
typename EmbeddingSpMDMKernelSignature<InType, IndexType, OffsetType, OutType>::Type
GenerateEmbeddingSpMDM(const std::int64_t block_size, bool has_weight, bool normalize_by_lengths, int prefetch = 16,
                       bool is_weight_positional = false, bool use_offsets = true, bool is_bf16_out = false,
                       bool is_bf16_in = false) {
  return GenerateEmbeddingSpMDMWithStrides<InType, IndexType, OffsetType, OutType, THREAD_LOCAL>(
      block_size, has_weight, normalize_by_lengths, prefetch, is_weight_positional, use_offsets, -1, -1, true, false,
      is_bf16_out, is_bf16_in);
}

// GenerateEmbeddingSpMDMNBitWithStrides (FbgemmEmbedding.h:151-174)
template <typename IndexType, typename OffsetType = std::int32_t, typename OutType = float, bool THREAD_LOCAL = false>
typename EmbeddingSpMDMKernelSignature<std::uint8_t, IndexType, OffsetType, OutType>::Type
GenerateEmbeddingSpMDMNBitWithStrides(const int input_bit_rate, const std::int64_t block_size, bool has_weight,
                                      bool normalize_by_lengths, int /*prefetch*/ = 16,
                                      bool is_weight_positional = false, bool use_offsets = true,
                                      std::int64_t output_stride = -1, std::int64_t input_stride = -1,
                                      bool scale_bias_last = true, const bool is_bf16_out = false,
                                      const bool no_bag = false, int output_bit_rate = -1) {
  if (input_bit_rate != 2 && input_bit_rate != 4) throw std::invalid_argument("fbgemm_amd: input_bit_rate must be 2 or 4");
  if (output_bit_rate == -1) output_bit_rate = 8 * (int)sizeof(OutType);
  fbgemm_amd_spmdm_config cfg{};
  cfg.no_bag = no_bag;
  cfg.weight_ty = input_bit_rate == 4 ? FBGEMM_AMD_INT4 : FBGEMM_AMD_INT2;
  // 4-bit rows to a 4-bit output (bytes copied) is the one no_bag form the reference has
  // (src/RefImplementations.cc:1466-1474); the call returns false for the others, as the reference does
  cfg.output_ty = (std::is_same_v<OutType, std::uint8_t> && output_bit_rate == 4) ? FBGEMM_AMD_INT4
                                                                                     : detail::output_ty<OutType>(is_bf16_out);
  if (no_bag && !(input_bit_rate == 4 && output_bit_rate == 4 && std::is_same_v<OutType, std::uint8_t>))
    return [](std::int64_t, std::int64_t, std::int64_t, const std::uint8_t*, const IndexType*, const OffsetType*,
              const float*, OutType*) { return false; };
  cfg.index_bits = detail::bits_of<IndexType>();
  cfg.offset_bits = detail::bits_of<OffsetType>();
  cfg.block_size = block_size;
  cfg.output_stride = output_stride;
  cfg.input_stride = input_stride;
  cfg.normalize_by_lengths = normalize_by_lengths;
  cfg.is_weight_positional = is_weight_positional;
  cfg.use_offsets = use_offsets;
  cfg.scale_bias_last = scale_bias_last;
  return [cfg, has_weight](std::int64_t output_size, std::int64_t index_size, std::int64_t data_size,
                           const std::uint8_t* input, const IndexType* indices, const OffsetType* offsets_or_lengths,
                           const float* weights, OutType* out) {
    return detail::run(cfg, output_size, index_size, data_size, input, indices, offsets_or_lengths, weights, out,
                       nullptr, has_weight);
  };
}

// GenerateEmbeddingSpMDMNBit (FbgemmEmbedding.h:124-140)
template <typename IndexType, typename OffsetType = std::int32_t, typename OutType = float>
typename EmbeddingSpMDMKernelSignature<std::uint8_t, IndexType, OffsetType, OutType>::Type
GenerateEmbeddingSpMDMNBit(int bit_rate, const std::int64_t block_size, bool has_weight, bool normalize_by_lengths,
                           int prefetch = 16, bool is_weight_positional = false, bool use_offsets = true) {
  return GenerateEmbeddingSpMDMNBitWithStrides<IndexType, OffsetType, OutType>(
      bit_rate, block_size, has_weight, normalize_by_lengths, prefetch, is_weight_positional, use_offsets);
}

// GenerateEmbeddingSpMDMFP8WithStrides (FbgemmEmbedding.h:185-203): rows of 8-bit floats, no scale/bias
template <typename IndexType, typename OffsetType = std::int32_t, typename OutType = float>
typename EmbeddingSpMDMKernelSignature<std::uint8_t, IndexType, OffsetType, OutType>::Type
GenerateEmbeddingSpMDMFP8WithStrides(const std::int64_t block_size, bool normalize_by_lengths,
                                     bool is_weight_positional = false, bool use_offsets = true,
                                     std::int64_t output_stride = -1, std::int64_t input_stride = -1,
                                     int exponent_bits = 4, int exponent_bias = 7, bool is_bf16_out = false) {
  fbgemm_amd_spmdm_config cfg{};
  cfg.weight_ty = FBGEMM_AMD_FP8;
  cfg.output_ty = detail::output_ty<OutType>(is_bf16_out);
  cfg.index_bits = detail::bits_of<IndexType>();
  cfg.offset_bits = detail::bits_of<OffsetType>();
  cfg.block_size = block_size;
  cfg.output_stride = output_stride;
  cfg.input_stride = input_stride;
  cfg.normalize_by_lengths = normalize_by_lengths;
  cfg.is_weight_positional = is_weight_positional;
  cfg.use_offsets = use_offsets;
  cfg.scale_bias_last = 1;
  cfg.fp8_exponent_bits = exponent_bits;
  cfg.fp8_exponent_bias = exponent_bias;
  // the reference's kernel takes the weights pointer as it comes (no has_weight flag)
  return [cfg](std::int64_t output_size, std::int64_t index_size, std::int64_t data_size, const std::uint8_t* input,
               const IndexType* indices, const OffsetType* offsets_or_lengths, const float* weights, OutType* out) {
    return detail::run(cfg, output_size, index_size, data_size, input, indices, offsets_or_lengths, weights, out,
                       nullptr, weights != nullptr);
  };
}

// GenerateEmbeddingSpMDMRowWiseSparse (FbgemmEmbedding.h:229-243)
template <typename InType, typename IndexType, typename OffsetType = std::int32_t>
typename EmbeddingSpMDMRowWiseSparseKernelSignature<InType, IndexType, OffsetType>::Type
GenerateEmbeddingSpMDMRowWiseSparse(const std::int64_t block_size, bool has_weight, bool normalize_by_lengths,
                                    int /*prefetch*/ = 16, bool is_weight_positional = false, bool use_offsets = true) {
  fbgemm_amd_spmdm_config cfg{};
  cfg.weight_ty = detail::weight_ty<InType>(false);
  cfg.output_ty = FBGEMM_AMD_FP32;
  cfg.index_bits = detail::bits_of<IndexType>();
  cfg.offset_bits = detail::bits_of<OffsetType>();
  cfg.block_size = block_size;
  cfg.output_stride = -1;
  cfg.input_stride = -1;
  cfg.normalize_by_lengths = normalize_by_lengths;
  cfg.is_weight_positional = is_weight_positional;
  cfg.use_offsets = use_offsets;
  cfg.scale_bias_last = true;
  return [cfg, has_weight](std::int64_t output_size, std::int64_t index_size, std::int64_t uncompressed_data_size,
                           const InType* input, const IndexType* indices, const OffsetType* offsets_or_lengths,
                           const float* weights, float* out, const std::int32_t* compressed_indices_table) {
    if (!compressed_indices_table) throw std::invalid_argument("fbgemm_amd: compressed_indices_table is null");
    return detail::run(cfg, output_size, index_size, uncompressed_data_size, input, indices, offsets_or_lengths,
                       weights, out, compressed_indices_table, has_weight);
  };
}

// GenerateEmbeddingSpMDMNBitRowWiseSparse (FbgemmEmbedding.h:250-262)
template <typename IndexType, typename OffsetType = std::int32_t>
typename EmbeddingSpMDMRowWiseSparseKernelSignature<std::uint8_t, IndexType, OffsetType>::Type
GenerateEmbeddingSpMDMNBitRowWiseSparse(int bit_rate, const std::int64_t block_size, bool has_weight,
                                        bool normalize_by_lengths, int /*prefetch*/ = 16,
                                        bool is_weight_positional = false, bool use_offsets = true) {
  if (bit_rate != 2 && bit_rate != 4) throw std::invalid_argument("fbgemm_amd: bit_rate must be 2 or 4");
  fbgemm_amd_spmdm_config cfg{};
  cfg.weight_ty = bit_rate == 4 ? FBGEMM_AMD_INT4 : FBGEMM_AMD_INT2;
  cfg.output_ty = FBGEMM_AMD_FP32;
  cfg.index_bits = detail::bits_of<IndexType>();
  cfg.offset_bits = detail::bits_of<OffsetType>();
  cfg.block_size = block_size;
  cfg.output_stride = -1;
  cfg.input_stride = -1;
  cfg.normalize_by_lengths = normalize_by_lengths;
  cfg.is_weight_positional = is_weight_positional;
  cfg.use_offsets = use_offsets;
  cfg.scale_bias_last = true;
  return [cfg, has_weight](std::int64_t output_size, std::int64_t index_size, std::int64_t uncompressed_data_size,
                           const std::uint8_t* input, const IndexType* indices, const OffsetType* offsets_or_lengths,
                           const float* weights, float* out, const std::int32_t* compressed_indices_table) {
    if (!compressed_indices_table) throw std::invalid_argument("fbgemm_amd: compressed_indices_table is null");
    return detail::run(cfg, output_size, index_size, uncompressed_data_size, input, indices, offsets_or_lengths,
                       weights, out, compressed_indices_table, has_weight);
  };
}

// ---- row-wise quantizers (include/fbgemm/QuantUtils.h:276-334 of the reference) ----
// Same names and argument lists; every pointer is a DEVICE pointer; the call
// returns when the work is done. `rowwise_min_max`, when given, is a device
// array of [input_rows][2] values (minimum, maximum) that take the place of
// each row's own extremes.

namespace detail {
template <typename T>
constexpr int float_ty() {
  if constexpr (std::is_same_v<T, float>) return FBGEMM_AMD_FP32;
  else if constexpr (std::is_same_v<T, float16> || std::is_same_v<T, std::uint16_t>) return FBGEMM_AMD_FP16;
  else if constexpr (std::is_same_v<T, bfloat16>) return FBGEMM_AMD_BF16;
  else static_assert(sizeof(T) == 0, "type must be float, float16, uint16_t or bfloat16");
}
inline void done(int rc) {
  if (rc < 0) throw std::runtime_error(std::string("fbgemm_amd: ") + fbgemm_amd_last_error());
  fbgemm_amd_stream_synchronize(stream_ref());
}
} // namespace detail

// compressed_indices_remap (FbgemmEmbedding.h:392-401): device pointers; returns when the work is done.
// As in the reference, nothing bounds the indices: every index must lie inside the mapping.
template <typename IndexType>
void compressed_indices_remap(std::int32_t offsets_numel, const IndexType* indices,
                              const std::int32_t* compressed_indices_mapping, const IndexType* offsets,
                              const float* weights, // optional, can be null
                              IndexType* out_indices, IndexType* out_offsets, float* out_weights) {
  detail::done(fbgemm_amd_compressed_indices_remap(offsets_numel, indices, detail::bits_of<IndexType>(),
                                                   compressed_indices_mapping, INT64_MAX, offsets, weights, out_indices,
                                                   out_offsets, out_weights, nullptr, stream_ref()));
}

template <typename InputType>
void FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(int bit_rate, const InputType* input, std::size_t input_rows,
                                                  int input_columns, std::uint8_t* output,
                                                  const InputType* rowwise_min_max = nullptr) {
  static_assert(!std::is_same_v<InputType, bfloat16>, "input is float or float16");
  const int epb = 8 / bit_rate;
  detail::done(fbgemm_amd_quantize_rowwise_min_max(input, detail::float_ty<InputType>(), (std::int64_t)input_rows,
                                                   input_columns, bit_rate, 0, FBGEMM_AMD_QLAYOUT_TRAILER,
                                                   (input_columns + epb - 1) / epb + 4, output, rowwise_min_max,
                                                   stream_ref()));
}

template <typename OutputType>
void FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf(int bit_rate, const std::uint8_t* input, std::size_t input_rows,
                                                  int input_columns, OutputType* output, bool scale_bias_last = true) {
  // input_columns counts the bytes of a fused row (QuantUtils.cc:758-760)
  const int cols = (input_columns - 4) * (8 / bit_rate);
  detail::done(fbgemm_amd_dequantize_rowwise(input, (std::int64_t)input_rows, input_columns, cols, bit_rate, 0,
                                             scale_bias_last ? FBGEMM_AMD_QLAYOUT_TRAILER : FBGEMM_AMD_QLAYOUT_TBE,
                                             detail::float_ty<OutputType>(), output, stream_ref()));
}

template <typename InputType>
void FloatOrHalfToFused8BitRowwiseQuantizedSBFloat(const InputType* input, std::size_t input_rows, int input_columns,
                                                   std::uint8_t* output, const InputType* rowwise_min_max = nullptr) {
  static_assert(!std::is_same_v<InputType, bfloat16>, "input is float or float16");
  detail::done(fbgemm_amd_quantize_rowwise_min_max(input, detail::float_ty<InputType>(), (std::int64_t)input_rows,
                                                   input_columns, 8, 1, FBGEMM_AMD_QLAYOUT_TRAILER, input_columns + 8,
                                                   output, rowwise_min_max, stream_ref()));
}

template <typename OutputType>
void Fused8BitRowwiseQuantizedSBFloatToFloatOrHalf(const std::uint8_t* input, std::size_t input_rows, int input_columns,
                                                   OutputType* output, const bool scale_bias_last = true,
                                                   const bool quant_padding_float_type = true) {
  if (scale_bias_last != quant_padding_float_type)
    throw std::invalid_argument("fbgemm_amd: rows are (data, fp32 scale, fp32 bias) or (fp16 scale, fp16 bias, data)");
  const int sb = quant_padding_float_type ? 8 : 4;
  detail::done(fbgemm_amd_dequantize_rowwise(input, (std::int64_t)input_rows, input_columns, input_columns - sb, 8,
                                             quant_padding_float_type ? 1 : 0,
                                             scale_bias_last ? FBGEMM_AMD_QLAYOUT_TRAILER : FBGEMM_AMD_QLAYOUT_TBE,
                                             detail::float_ty<OutputType>(), output, stream_ref()));
}

} // namespace fbgemm_amd
