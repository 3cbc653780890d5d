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
void oracle_quantize_rowwise_min_max(const void* input, int half_in, int64_t rows, int32_t cols, int32_t bit_rate,
                                     int32_t sb_float, int32_t layout, int64_t out_stride, uint8_t* output,
                                     const void* min_max);

void oracle_quantize_rowwise(const void* input, int half_in, int64_t rows, int32_t cols, int32_t bit_rate,
                             int32_t sb_float, int32_t layout, int64_t out_stride, uint8_t* output) {
  oracle_quantize_rowwise_min_max(input, half_in, rows, cols, bit_rate, sb_float, layout, out_stride, output, 0);
}

/*
 * min_max, when not null: [rows][2] values of the input's type, (minimum, maximum), used in place
 * of the row's own extremes (src/QuantUtilsAvx2.cc:1605-1628, :1831-1853 -- only the reference's
 * vector routines take them, its scalar *Ref routines do not). An element outside them:
 *   fp16-pair formats: clamped to 0 .. 2^bit_rate - 1 at every column (:1719-1722 for whole groups
 *     of 32 columns, :1768-1773 for the rest); what is clamped is the rounded value as a 32-bit
 *     integer, which for a value beyond 32 bits is 0x80000000 in the whole groups of 32 columns
 *     of the 2- and 4-bit formats and the low half of the 64-bit integer in the other columns;
 *   8-bit fp32-pair format: columns in the leading whole groups of 32 saturate to 0 .. 255 (the
 *     signed 32->16 and unsigned 16->8 packs, :1930-1932); the columns behind keep the low byte
 *     of the rounded 32-bit integer (:1938-1945 byte shuffle, :1947-1950 lrintf to uint8_t). A
 *     value that does not fit 32 bits (or a NaN) converts to 0x80000000, which both rules turn
 *     into 0.
 */
void oracle_quantize_rowwise_min_max(const void* input, int half_in, int64_t rows, int32_t cols, int32_t bit_rate,
                                     int32_t sb_float, int32_t layout, int64_t out_stride, uint8_t* output,
                                     const void* min_max) {
  const int epb = 8 / bit_rate;
  const int data_bytes = (cols + epb - 1) / epb;
  const int maxq = (1 << bit_rate) - 1;
  for (int64_t r = 0; r < rows; ++r) {
    uint8_t* out_row = output + r * out_stride;
    uint8_t* data = layout == LAYOUT_TBE ? out_row + 4 : out_row;
    uint8_t* sb = layout == LAYOUT_TBE ? out_row : out_row + data_bytes;
    float minimum, maximum;
    row_extremes(input, half_in, r * (int64_t)cols, cols, &minimum, &maximum);
    if (min_max) {
      minimum = in_elem(min_max, half_in, 2 * r);
      maximum = in_elem(min_max, half_in, 2 * r + 1);
    }
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
      for (int j = 0; j < cols; ++j) {
        const float v = rintf((in_elem(input, half_in, r * (int64_t)cols + j) - minimum) * inverse_scale);
        if (!min_max) {
          data[j] = (uint8_t)lrintf(v);
        } else if (!(fabsf(v) < 2147483648.0f)) {
          data[j] = 0; /* the conversion yields 0x80000000: saturates to 0, and its low byte is 0 */
        } else if (j < cols / 32 * 32) {
          data[j] = (uint8_t)(v > 0.0f ? (v > 255.0f ? 255.0f : v) : 0.0f);
        } else {
          data[j] = (uint8_t)(int32_t)v;
        }
      }
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
        const float v = rintf((x - minimum) * inverse_scale);
        int32_t q;
        if (!min_max) {
          q = (int32_t)lrintf(v);
        } else if (bit_rate < 8 && j < cols / 32 * 32) {
          /* whole groups of 32 columns, 2 and 4 bits: the 32-bit conversion yields 0x80000000 for
           * what does not fit (a NaN too), which the packs saturate to 0 (:1697-1722) */
          q = fabsf(v) < 2147483648.0f ? (int32_t)v : INT32_MIN;
        } else {
          /* the other columns: lrintf's 64-bit result cut to its low 32 bits by std::min<int>
           * (:1768-1773); 0x8000000000000000 for what does not fit 64 bits */
          q = fabsf(v) < 9223372036854775808.0f ? (int32_t)(uint32_t)(uint64_t)(int64_t)v : 0;
        }
        int qi = q < maxq ? q : maxq;
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

/* ---- fp32 -> 8-bit float (hfp8) ----------------------------------------------
 * float_to_hfp8 (fbgemm_gpu/include/fbgemm_gpu/quantize_ops_utils.h:29-81), which is
 * FloatToFloat8_ref (src/RefImplementations.cc:126-182) with max_pos as an argument:
 * clamp |x| to max_pos; normal range: round to 7 - ebits mantissa bits by adding and
 * subtracting a power of two 23 - mbits binades above x (fp32's own round-to-nearest-
 * even does the rounding), re-bias the exponent, shift the 7 code bits into place;
 * below the smallest normal 2^(1 - bias): add 2^(24 - bias - mbits), whose low bits
 * then are the code. The sign goes to bit 7. Pinned by tests/test_hfp8_oracle.py:
 * against the reference's FloatToFloat8_ref compiled from its sources, and against
 * "nearest of the 128 representable magnitudes, ties to the even code, saturating".
 * The decoder is oracle_float8_to_float (embedding_oracle.c). */
uint8_t oracle_float_to_hfp8(float x, int ebits, int exponent_bias, float max_pos) {
  const int mbits = 7 - ebits;
  union { uint32_t i; float f; } v, bouncer, smallest_normal;
  v.f = x;
  const uint32_t sign = v.i & 0x80000000u;
  v.i &= 0x7fffffffu;
  v.f = fminf(v.f, max_pos);
  smallest_normal.i = (uint32_t)(127 - exponent_bias + 1) << 23;
  if (v.f >= smallest_normal.f) {
    bouncer.i = (v.i & 0xff800000u) + ((uint32_t)(23 - mbits) << 23);
    volatile float t = bouncer.f + v.f; /* each step rounded to fp32 */
    v.f = t - bouncer.f;
    v.i = (v.i - ((uint32_t)(127 - exponent_bias) << 23)) << (8 - ebits);
    v.i = (v.i | sign) >> 24;
  } else {
    bouncer.i = (uint32_t)(127 + (23 + (1 - exponent_bias - mbits))) << 23;
    v.f = bouncer.f + v.f;
    v.i = v.i | (sign >> 24);
  }
  return (uint8_t)v.i;
}

/* FloatToFloat8_ref's own max_pos (src/RefImplementations.cc:131-132) */
float oracle_hfp8_max_pos(int ebits, int exponent_bias) {
  return (float)((double)(1 << ((1 << ebits) - 2 - exponent_bias)) * (2.0 - pow(2.0, ebits - 7)));
}

void oracle_float_to_hfp8_array(const float* in, uint8_t* out, int64_t n, int ebits, int exponent_bias, float max_pos) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_float_to_hfp8(in[i], ebits, exponent_bias, max_pos);
}
