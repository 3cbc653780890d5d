/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the row-wise quantizers that
 * produce (and read back) the row formats the embedding-bag lookup consumes.
 *
 * A plain-C restatement of the reference's scalar routines. Nothing in the
 * shipped library links, loads or calls this file.
 *
 * Parity status: PINNED. tests/test_quantize_oracle.py checks every function
 * bit for bit against the reference's own routines compiled from its sources
 * (oracle/_ref/libfbgemm_ref_quant.so: src/QuantUtils.cc, both the *Ref
 * functions and the AVX2 entry points), and against what the arithmetic fixes:
 * a constant row quantizes to zeros with scale 1 (N-bit) / 0 (8-bit), a row
 * holding exactly the 2^bits grid points min + k * scale round-trips exactly,
 * quantize -> dequantize errs by at most scale / 2 (+ the fp16 rounding of the
 * bias), the first of two equal extremes decides the sign of a zero bias.
 *
 * Reference files followed:
 *   src/QuantUtils.cc:534-611   FloatOrHalfToFusedNBitRowwiseQuantizedSBHalfRef
 *   src/QuantUtils.cc:677-718   FloatOrHalfToFused8BitRowwiseQuantizedSBFloatRef
 *   src/QuantUtils.cc:743-789   FusedNBitRowwiseQuantizedSBHalfToFloatOrHalfRef
 *   src/QuantUtils.cc:847-892   Fused8BitRowwiseQuantizedSBFloatToFloatOrHalfRef
 *   fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:20-72  quantize_embs (row re-layout)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

float oracle_half2float(uint16_t h);
uint16_t oracle_float2half_rn(float f);
uint16_t oracle_float2bf16(float f);

enum { ST_FP32 = 0, ST_FP16 = 1, ST_BF16 = 5 };
enum { LAYOUT_TRAILER = 0, LAYOUT_TBE = 1 };

static float in_elem(const void* in, int half_in, int64_t i) {
  return half_in ? oracle_half2float(((const uint16_t*)in)[i]) : ((const float*)in)[i];
}

/* the first smallest / largest element (std::ranges::min_element / max_element) */
static void row_extremes(const void* in, int half_in, int64_t base, int cols, float* mn, float* mx) {
  float lo = in_elem(in, half_in, base), hi = lo;
  for (int j = 1; j < cols; ++j) {
    const float x = in_elem(in, half_in, base + j);
    if (x < lo) lo = x;
    if (hi < x) hi = x;
  }
  *mn = lo;
  *mx = hi;
}

/*
 * One routine for the three producers.
 *   sb_float = 0: N-bit rule with fp16 scale / bias (bit_rate 2, 4, 8)
 *   sb_float = 1: 8-bit rule with fp32 scale / bias
 *   layout TRAILER: elements, then (scale, bias); TBE: fp16 (scale, bias), then
 *   elements (an fp32 pair is rounded to fp16 on the way, as quantize_embs does).
 * Bytes of a row beyond what the format defines are left alone.
 */
void oracle_quantize_rowwise(const void* input, int half_in, int64_t rows, int32_t cols, int32_t bit_rate,
                             int32_t sb_float, int32_t layout, int64_t out_stride, uint8_t* output) {
  const int epb = 8 / bit_rate;
  const int data_bytes = (cols + epb - 1) / epb;
  const int maxq = (1 << bit_rate) - 1;
  for (int64_t r = 0; r < rows; ++r) {
    uint8_t* out_row = output + r * out_stride;
    uint8_t* data = layout == LAYOUT_TBE ? out_row + 4 : out_row;
    uint8_t* sb = layout == LAYOUT_TBE ? out_row : out_row + data_bytes;
    float minimum, maximum;
    row_extremes(input, half_in, r * (int64_t)cols, cols, &minimum, &maximum);
    if (sb_float) {
      const float range = maximum - minimum;
      const float scale = range / 255.0f;
      const float inverse_scale = 255.0f / (range + 1e-8f);
      if (layout == LAYOUT_TBE) {
        const uint16_t s16 = oracle_float2half_rn(scale), b16 = oracle_float2half_rn(minimum);
        memcpy(sb, &s16, 2);
        memcpy(sb + 2, &b16, 2);
      } else {
        memcpy(sb, &scale, 4);
        memcpy(sb + 4, &minimum, 4);
      }
      for (int j = 0; j < cols; ++j)
        data[j] = (uint8_t)lrintf((in_elem(input, half_in, r * (int64_t)cols + j) - minimum) * inverse_scale);
    } else {
      const uint16_t min16 = oracle_float2half_rn(minimum);
      minimum = oracle_half2float(min16);
      const float range = maximum - minimum;
      float scale = range == 0 ? 1.0f : range / (float)maxq;
      scale = oracle_half2float(oracle_float2half_rn(scale));
      if (scale == 0) scale = 1.0f;
      float inverse_scale = 1.0f / scale;
      if (isinf(inverse_scale)) {
        scale = 1.0f;
        inverse_scale = 1.0f;
      }
      const uint16_t s16 = oracle_float2half_rn(scale);
      memcpy(sb, &s16, 2);
      memcpy(sb + 2, &min16, 2);
      for (int j = 0; j < cols; ++j) {
        const float x = in_elem(input, half_in, r * (int64_t)cols + j);
        long q = lrintf((x - minimum) * inverse_scale);
        int qi = (int)q < maxq ? (int)q : maxq;
        qi = qi > 0 ? qi : 0;
        if (j % epb == 0) data[j / epb] = (uint8_t)qi;
        else data[j / epb] |= (uint8_t)(qi << ((j % epb) * bit_rate));
      }
    }
  }
}

void oracle_dequantize_rowwise(const uint8_t* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t bit_rate,
                               int32_t sb_float, int32_t layout, int32_t output_ty, void* output) {
  const int epb = 8 / bit_rate;
  const int data_bytes = (cols + epb - 1) / epb;
  for (int64_t r = 0; r < rows; ++r) {
    const uint8_t* in_row = input + r * in_stride;
    const uint8_t* data = layout == LAYOUT_TBE ? in_row + 4 : in_row;
    const uint8_t* sb = layout == LAYOUT_TBE ? in_row : in_row + data_bytes;
    float scale, bias;
    if (sb_float) {
      memcpy(&scale, sb, 4);
      memcpy(&bias, sb + 4, 4);
    } else {
      uint16_t s16, b16;
      memcpy(&s16, sb, 2);
      memcpy(&b16, sb + 2, 2);
      scale = oracle_half2float(s16);
      bias = oracle_half2float(b16);
    }
    for (int j = 0; j < cols; ++j) {
      uint8_t q = data[j / epb];
      q >>= (j % epb) * bit_rate;
      q &= (uint8_t)((1 << bit_rate) - 1);
      const float v = (float)((double)scale * q + (double)bias);
      const int64_t o = r * (int64_t)cols + j;
      if (output_ty == ST_FP32) ((float*)output)[o] = v;
      else if (output_ty == ST_BF16) ((uint16_t*)output)[o] = oracle_float2bf16(v);
      else ((uint16_t*)output)[o] = oracle_float2half_rn(v);
    }
  }
}
