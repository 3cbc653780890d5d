// TEST INFRASTRUCTURE ONLY -- extern "C" entry points over the reference's own
// row-wise quantizers (src/QuantUtils.cc, src/QuantUtilsAvx2.cc), compiled from the
// reference tree where it lies. Used to pin oracle/quantize_oracle.c; never loaded
// by the library.
#include <cstddef>
#include <cstdint>

#include "fbgemm/QuantUtils.h"
#include "fbgemm/QuantUtilsAvx2.h"

using fbgemm::bfloat16;
using fbgemm::float16;

extern "C" {

// the scalar *Ref routines: what the reference's own tests hold its vector code to
void ref_quantize_nbit(int bit_rate, const void* in, int half_in, int64_t rows, int cols, uint8_t* out) {
  if (half_in) fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfRef<float16>(bit_rate, (const float16*)in, rows, cols, out);
  else fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfRef<float>(bit_rate, (const float*)in, rows, cols, out);
}

void ref_quantize_8bit(const void* in, int half_in, int64_t rows, int cols, uint8_t* out) {
  if (half_in) fbgemm::FloatOrHalfToFused8BitRowwiseQuantizedSBFloatRef<float16>((const float16*)in, rows, cols, out);
  else fbgemm::FloatOrHalfToFused8BitRowwiseQuantizedSBFloatRef<float>((const float*)in, rows, cols, out);
}

// the AVX2 routines, the only ones that take caller-supplied extremes (min_max may be null)
void ref_quantize_nbit_avx2(int bit_rate, const void* in, int half_in, int64_t rows, int cols, uint8_t* out,
                            const void* min_max) {
  if (half_in) {
    const float16* x = (const float16*)in;
    const float16* mm = (const float16*)min_max;
    if (bit_rate == 2) fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float16, 2>(x, rows, cols, out, mm);
    else if (bit_rate == 4) fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float16, 4>(x, rows, cols, out, mm);
    else fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float16, 8>(x, rows, cols, out, mm);
  } else {
    const float* x = (const float*)in;
    const float* mm = (const float*)min_max;
    if (bit_rate == 2) fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float, 2>(x, rows, cols, out, mm);
    else if (bit_rate == 4) fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float, 4>(x, rows, cols, out, mm);
    else fbgemm::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfAvx2<float, 8>(x, rows, cols, out, mm);
  }
}

void ref_quantize_8bit_avx2(const void* in, int half_in, int64_t rows, int cols, uint8_t* out, const void* min_max) {
  if (half_in) fbgemm::FloatOrHalfToFused8BitRowwiseQuantizedSBFloatAvx2<float16>((const float16*)in, rows, cols, out, (const float16*)min_max);
  else fbgemm::FloatOrHalfToFused8BitRowwiseQuantizedSBFloatAvx2<float>((const float*)in, rows, cols, out, (const float*)min_max);
}

// out_ty: 0 fp32, 1 fp16, 5 bf16; input_columns counts the bytes of a fused row
void ref_dequantize_nbit(int bit_rate, const uint8_t* in, int64_t rows, int input_columns, int out_ty, void* out) {
  if (out_ty == 0) fbgemm::FusedNBitRowwiseQuantizedSBHalfToFloatOrHalfRef<float>(bit_rate, in, rows, input_columns, (float*)out, true);
  else if (out_ty == 1) fbgemm::FusedNBitRowwiseQuantizedSBHalfToFloatOrHalfRef<float16>(bit_rate, in, rows, input_columns, (float16*)out, true);
  else fbgemm::FusedNBitRowwiseQuantizedSBHalfToFloatOrHalfRef<bfloat16>(bit_rate, in, rows, input_columns, (bfloat16*)out, true);
}

void ref_dequantize_8bit(const uint8_t* in, int64_t rows, int input_columns, int out_ty, void* out) {
  if (out_ty == 0) fbgemm::Fused8BitRowwiseQuantizedSBFloatToFloatOrHalfRef<float>(in, rows, input_columns, (float*)out, true, true);
  else if (out_ty == 1) fbgemm::Fused8BitRowwiseQuantizedSBFloatToFloatOrHalfRef<float16>(in, rows, input_columns, (float16*)out, true, true);
  else fbgemm::Fused8BitRowwiseQuantizedSBFloatToFloatOrHalfRef<bfloat16>(in, rows, input_columns, (bfloat16*)out, true, true);
}

} // extern "C"
