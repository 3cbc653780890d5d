/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the quantized embedding-bag path.
 *
 * A plain-C restatement of the reference's scalar algorithms. Nothing in the
 * shipped library links, loads or calls this file: it exists so that tests,
 * the smoke check and the benchmark's CPU leg can check the HIP kernels
 * against an independent evaluation of the same arithmetic.
 *
 * Parity status of every function here: PINNED. Each one is cross-checked
 * bit-for-bit in tests/ against the reference's own scalar implementation
 * compiled from its sources (oracle/_ref), against closed forms
 * (scale=1/bias=0 integer sums, all-ones rows counting kept indices,
 * single-row fma identities), against numpy's IEEE half conversion over all
 * 65536 half patterns, and against a float64 brute-force evaluation.
 *
 * Reference files followed (paths relative to the reference tree):
 *   src/RefImplementations.cc:1196-1425  EmbeddingSpMDM_ref (8-bit, fp16, fp32 rows)
 *   src/RefImplementations.cc:1427-1541  EmbeddingSpMDMNBit_ref (int4 / int2 rows)
 *   src/RefImplementations.cc:1235-1288,1352-1376,1466-1484  the no_bag branches of both
 *   src/RefImplementations.cc:184-214,1544-1616  Float8ToFloat_ref, EmbeddingSpMDMFP8_ref
 *   src/RefImplementations.cc:1617-1822  row-wise-sparse variants
 *   src/RefImplementations.cc:2308-2333  compressed_indices_remap_ref
 *   src/RefImplementations.h:428-453     float <-> storage conversions
 *   include/fbgemm/FloatConversion.h:82-217,229-315  fp16 RNE, half->float, bf16
 *   fbgemm_gpu/include/fbgemm_gpu/embedding_common.h:20-48,189-225  enums, row sizes
 *   fbgemm_gpu/codegen/inference/embedding_forward_quantized_cpu_template.cpp:208-520,605-659
 *                                        table-batched forward loop, pruned_array_lookup
 *   fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update_cpu.cpp:25-70,199-251
 *                                        emb_inplace_update, pruned_array_lookup_from_row_idx
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- weight / output element types (same numbering as the reference's
 *      SparseType, embedding_common.h:20-32) ------------------------------ */
enum { ST_FP32 = 0, ST_FP16 = 1, ST_INT8 = 2, ST_INT4 = 3, ST_INT2 = 4, ST_BF16 = 5 };

/* ---- scalar float conversions ------------------------------------------ */

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE half -> float, exact (FloatConversion.h:229-279). */
float oracle_half2float(uint16_t h) {
  uint32_t sign = (uint32_t)(h >> 15) & 1u;
  uint32_t exp = (uint32_t)(h >> 10) & 0x1fu;
  uint32_t man = ((uint32_t)h & 0x3ffu) << 13;
  if (exp == 0x1f) {
    /* the portable reference canonicalises NaN; the F16C path it normally
       uses keeps sign and payload. Outputs only ever carry finite rows, so
       follow the hardware (payload-preserving, quieted) behaviour. */
    if (man) return u2f((sign << 31) | 0x7f800000u | man | 0x00400000u);
    return u2f((sign << 31) | 0x7f800000u);
  }
  if (exp == 0) {
    if (man == 0) return u2f(sign << 31);
    exp = 127 - 15 + 1;
    uint32_t top;
    do {
      top = man & (1u << 22);
      man <<= 1;
      --exp;
    } while (!top);
    man &= 0x7fffffu;
    return u2f((sign << 31) | (exp << 23) | man);
  }
  return u2f((sign << 31) | ((exp + 112u) << 23) | man);
}

/* float -> IEEE half, round to nearest even, denormals kept, overflow to inf
 * (FloatConversion.h:82-217 with Src=single, Tgt=half). */
uint16_t oracle_float2half_rn(float f) {
  uint32_t v = f2u(f);
  uint32_t sexp = v & 0x7f800000u;
  uint32_t sman = v & 0x007fffffu;
  uint16_t sign = (uint16_t)((v >> 16) & 0x8000u);
  if (sexp == 0) return sign; /* zero or fp32 denormal: far below half range */
  int e = (int)(sexp >> 23) - 127;
  if (e < -14) {
    int shift = -14 - e;
    if (shift > 11) return sign;
    uint32_t m1 = sman | 0x00800000u;
    uint16_t tm = (uint16_t)(m1 >> (13 + shift));
    uint32_t half = 1u << (13 + shift - 1);
    uint32_t rem = m1 & ((half << 1) - 1);
    if (rem > half || (rem == half && (tm & 1))) tm += 1;
    return sign | tm;
  }
  if (e > 15) {
    if (e == 128 && sman != 0) {
      return sign | 0x7c00u | (uint16_t)(sman >> 13) | 0x0200u;
    }
    return sign | 0x7c00u;
  }
  uint16_t tm = (uint16_t)(sman >> 13);
  uint16_t te = (uint16_t)((e + 15) << 10);
  uint32_t rem = sman & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (tm & 1))) {
    if (tm < 0x3ff) {
      tm += 1;
    } else {
      tm = 0;
      te += 0x0400u;
    }
  }
  return sign | te | tm;
}

/* float -> bf16 the way the reference writes it: add half an ulp to the bit
 * pattern and truncate (FloatConversion.h:312-315). Not IEEE RNE on ties. */
uint16_t oracle_float2bf16(float f) {
  return (uint16_t)((f2u(f) + 0x8000u) >> 16);
}

float oracle_bf162float(uint16_t b) { return u2f((uint32_t)b << 16); }

static void store_out(void* out, int out_ty, int64_t pos, float v) {
  if (out_ty == ST_FP32) ((float*)out)[pos] = v;
  else if (out_ty == ST_FP16) ((uint16_t*)out)[pos] = oracle_float2half_rn(v);
  else ((uint16_t*)out)[pos] = oracle_float2bf16(v);
}

static int64_t read_index(const void* p, int is64, int64_t i) {
  return is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

/* ---- row-size arithmetic (embedding_common.h:189-225) ------------------ */

int32_t oracle_unpadded_row_bytes(int32_t dim, int ty, int32_t scale_bias_bytes) {
  switch (ty) {
    case ST_FP32: return dim * 4;
    case ST_FP16: return dim * 2;
    case ST_INT8: return dim + scale_bias_bytes;
    case ST_INT4: return dim / 2 + scale_bias_bytes;
    case ST_INT2: return dim / 4 + scale_bias_bytes;
    default: return 0;
  }
}

int32_t oracle_padded_row_bytes(int32_t dim, int ty, int32_t row_alignment,
                                int32_t scale_bias_bytes) {
  uint64_t r = (uint64_t)oracle_unpadded_row_bytes(dim, ty, scale_bias_bytes);
  uint64_t a = (uint64_t)row_alignment;
  return (int32_t)(((r + a - 1) / a) * a);
}

/* ---- the pooled lookup --------------------------------------------------
 *
 * One function covers every row format on the path; `in_ty` selects it.
 *   ST_INT8: D bytes + (fp32 scale, fp32 bias) after them when
 *            scale_bias_last, or (fp16 scale, fp16 bias) before them when not.
 *   ST_INT4 / ST_INT2: ceil(D / elems_per_byte) packed bytes, element j sits
 *            in byte j / epb at bit (j % epb) * bits; fp16 scale and bias
 *            after (scale_bias_last) or before the packed bytes.
 *   ST_FP16 / ST_BF16 / ST_FP32: plain rows, no scale/bias.
 * input_stride is counted in elements of the storage type (bytes for the
 * integer formats, halfs for fp16/bf16, floats for fp32), as in the
 * reference's templates. -1 picks the dense default.
 *
 * When `remap` is non-null the call follows the row-wise-sparse variants:
 * the bound check applies to the logical index, the physical row is
 * remap[logical], -1 there skips the row, and the layout is the trailer one.
 *
 * Returns 1 on success and 0 where the reference returns false.
 */
int oracle_embedding_spmdm(
    int in_ty, int64_t block_size, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* input, const void* indices, int idx64,
    const void* offsets_or_lengths, int off64, const float* weights,
    int normalize_by_lengths, void* out, int out_ty, int is_weight_positional,
    int use_offsets, int64_t output_stride, int64_t input_stride,
    int scale_bias_last, const int32_t* remap) {
  const int quantised = in_ty == ST_INT8 || in_ty == ST_INT4 || in_ty == ST_INT2;
  const int bits = in_ty == ST_INT8 ? 8 : in_ty == ST_INT4 ? 4 : 2;
  const int epb = 8 / bits;
  const int64_t packed = (block_size + epb - 1) / epb;
  const uint8_t* in8 = (const uint8_t*)input;
  int64_t head = 0; /* bytes of scale/bias in front of the data */

  if (output_stride == -1) output_stride = block_size;
  if (quantised) {
    int64_t sb;
    if (in_ty == ST_INT8) sb = scale_bias_last ? 8 : 4;
    else sb = 4;
    if (input_stride == -1) input_stride = packed + sb;
    head = scale_bias_last ? 0 : sb;
  } else if (input_stride == -1) {
    input_stride = block_size;
  }

  float* buf = (float*)malloc(sizeof(float) * (size_t)(block_size > 0 ? block_size : 1));
  int64_t current = 0;
  int ok = 1;
  for (int64_t m = 0; m < output_size && ok; ++m) {
    for (int64_t j = 0; j < block_size; ++j) buf[j] = 0.0f;
    /* the reference keeps the bag length in a 32-bit int */
    int len = use_offsets
        ? (int)(read_index(offsets_or_lengths, off64, m + 1) -
                read_index(offsets_or_lengths, off64, m))
        : (int)read_index(offsets_or_lengths, off64, m);
    if (current + len > index_size) { ok = 0; break; }
    for (int i = 0; i < len; ++i, ++current) {
      int64_t idx = read_index(indices, idx64, current);
      if (remap) {
        if (idx < 0 || idx >= data_size) { ok = 0; break; }
        idx = (int64_t)remap[idx];
        if (idx == -1) continue;
      } else {
        if (!scale_bias_last && idx == -1) continue; /* pruned row, TBE layouts only */
        if (idx < 0 || idx >= data_size) { ok = 0; break; }
      }
      float w = 1.0f;
      if (weights) w = weights[is_weight_positional ? i : current];

      if (quantised) {
        const uint8_t* row = in8 + input_stride * idx;
        float scale, bias;
        if (in_ty == ST_INT8 && scale_bias_last) {
          float sb[2];
          memcpy(sb, row + block_size, 8);
          scale = w * sb[0];
          bias = w * sb[1];
        } else {
          uint16_t sb[2];
          memcpy(sb, row + (scale_bias_last ? packed : 0), 4);
          scale = w * oracle_half2float(sb[0]);
          bias = w * oracle_half2float(sb[1]);
        }
        const uint8_t* q = row + head;
        for (int64_t j = 0; j < block_size; ++j) {
          uint8_t v = q[j / epb];
          v >>= (j % epb) * bits;
          v &= (uint8_t)((1 << bits) - 1);
          buf[j] = fmaf(scale, (float)v, buf[j] + bias);
        }
      } else if (in_ty == ST_FP32) {
        const float* row = (const float*)input + input_stride * idx;
        for (int64_t j = 0; j < block_size; ++j) buf[j] = fmaf(w, row[j], buf[j]);
      } else {
        const uint16_t* row = (const uint16_t*)input + input_stride * idx;
        for (int64_t j = 0; j < block_size; ++j) {
          float x = in_ty == ST_BF16 ? oracle_bf162float(row[j]) : oracle_half2float(row[j]);
          buf[j] = fmaf(w, x, buf[j]);
        }
      }
    }
    if (!ok) break;
    if (normalize_by_lengths && len) {
      float s = 1.f / (float)len;
      for (int64_t j = 0; j < block_size; ++j) buf[j] *= s;
    }
    for (int64_t j = 0; j < block_size; ++j) store_out(out, out_ty, m * output_stride + j, buf[j]);
  }
  free(buf);
  if (!ok) return 0;
  return current == index_size;
}

/* ---- compacting remap (RefImplementations.cc:2308-2333) ----------------
 * Drops pruned entries, rewrites offsets (and weights). The reference walks
 * k with a 32-bit counter; keep that. */
void oracle_compressed_indices_remap(
    int32_t offsets_len, const void* indices, int idx64, const int32_t* mapping,
    const void* offsets, const float* weights, void* out_indices,
    void* out_offsets, float* out_weights) {
  int64_t j = 0;
  int64_t first = read_index(offsets, idx64, 0);
  if (idx64) ((int64_t*)out_offsets)[0] = first; else ((int32_t*)out_offsets)[0] = (int32_t)first;
  for (int i = 1; i < offsets_len; ++i) {
    for (int32_t k = (int32_t)read_index(offsets, idx64, i - 1);
         k < read_index(offsets, idx64, i); ++k) {
      int32_t m = mapping[read_index(indices, idx64, k)];
      if (m != -1) {
        if (idx64) ((int64_t*)out_indices)[j] = m; else ((int32_t*)out_indices)[j] = m;
        if (weights) out_weights[j] = weights[k];
        ++j;
      }
    }
    if (idx64) ((int64_t*)out_offsets)[i] = j; else ((int32_t*)out_offsets)[i] = (int32_t)j;
  }
}

/* ---- position-preserving remap (…_cpu_template.cpp:605-659) ------------
 * dense[i] = remap[start_t + idx[i]] for tables that own a mapping, a plain
 * copy for tables that do not. remap entries are int32 or int64. */
void oracle_pruned_array_lookup(
    int32_t T, int32_t B, const void* indices, const void* offsets, int idx64,
    const void* remap, int remap64, const int64_t* remap_offsets, void* dense) {
  for (int32_t t = 0; t < T; ++t) {
    int64_t rs = remap_offsets[t], re = remap_offsets[t + 1];
    int64_t is = read_index(offsets, idx64, (int64_t)t * B);
    int64_t ie = read_index(offsets, idx64, (int64_t)(t + 1) * B);
    for (int64_t i = is; i < ie; ++i) {
      int64_t v = read_index(indices, idx64, i);
      if (re - rs > 0) v = read_index(remap, remap64, rs + v);
      if (idx64) ((int64_t*)dense)[i] = v; else ((int32_t*)dense)[i] = (int32_t)v;
    }
  }
}

/* ---- in-place row update (fbgemm_gpu/src/embedding_inplace_ops/
 *      embedding_inplace_update_cpu.cpp:25-70) --------------------------------
 * Update n overwrites the padded row update_row_idx[n] of table
 * update_table_idx[n] with the bytes at update_weights + update_offsets[n];
 * updates are applied in order (the last one of a row wins). The buffer is
 * chosen by the table's placement: 0 = the first weights buffer. */
void oracle_emb_inplace_update(
    uint8_t* dev_weights, uint8_t* uvm_weights, const int32_t* weights_placements,
    const int64_t* weights_offsets, const uint8_t* weights_tys, const int32_t* D_offsets,
    const uint8_t* update_weights, const int32_t* update_table_idx, const void* update_row_idx,
    int idx64, const int64_t* update_offsets, int64_t n_updates, int64_t row_alignment) {
  for (int64_t n = 0; n < n_updates; ++n) {
    int32_t t = update_table_idx[n];
    int64_t row = read_index(update_row_idx, idx64, n);
    int32_t D = D_offsets[t + 1] - D_offsets[t];
    int32_t D_bytes = oracle_padded_row_bytes(D, weights_tys[t], (int32_t)row_alignment, 4);
    uint8_t* base = weights_placements[t] == 0 ? dev_weights : uvm_weights;
    memcpy(base + weights_offsets[t] + (int64_t)D_bytes * row, update_weights + update_offsets[n], (size_t)D_bytes);
  }
}

/* pruned_array_lookup_from_row_idx (embedding_inplace_update_cpu.cpp:199-251):
 * the rows of an update through the pruning arrays; tables without a mapping
 * keep their rows. */
void oracle_pruned_array_lookup_from_row_idx(
    int64_t n, const void* update_row_idx, int idx64, const int32_t* update_table_idx,
    const void* remap, int remap64, const int64_t* remap_offsets, void* dense) {
  for (int64_t i = 0; i < n; ++i) {
    int32_t t = update_table_idx[i];
    int64_t v = read_index(update_row_idx, idx64, i);
    int64_t rs = remap_offsets[t], re = remap_offsets[t + 1];
    if (re - rs > 0) v = read_index(remap, remap64, rs + v);
    if (idx64) ((int64_t*)dense)[i] = v; else ((int32_t*)dense)[i] = (int32_t)v;
  }
}

/* ---- table-batched forward (…_cpu_template.cpp:208-520) ----------------
 *
 * Runs the pooled lookup once per table on that table's slice of the
 * (table, bag)-ordered offsets, writing the table's column block of the
 * [B, total_D] output. Scale/bias sit in front of the row as two halfs,
 * rows are padded to row_alignment, -1 indices are skipped.
 *
 * The number of rows of table t is not an argument of the reference
 * operator: it is inferred as (next distinct weights offset - this offset) /
 * row bytes, the last table being bounded by the size of the weights buffer.
 * The same inference is made here so that the same indices are rejected.
 *
 * Returns 0 on success, or 1 + t for the first table whose lookup failed
 * (where the reference raises).
 */
static int cmp_i64(const void* a, const void* b) {
  int64_t x = *(const int64_t*)a, y = *(const int64_t*)b;
  return x < y ? -1 : x > y;
}

int oracle_tbe_forward(
    const uint8_t* dev_weights, int64_t weights_numel, const int64_t* weights_offsets,
    const uint8_t* weights_tys, const int32_t* D_offsets, int32_t T, int64_t total_D,
    const void* indices, const void* offsets, int idx64, int64_t offsets_numel,
    int pooling_mode, const float* indice_weights, int out_ty, int64_t row_alignment,
    void* output) {
  int32_t B = (int32_t)((offsets_numel - 1) / T);
  if (B == 0) return 0;
  size_t esz = out_ty == ST_FP32 ? 4 : 2;
  memset(output, 0, esz * (size_t)B * (size_t)total_D);

  int64_t* phys = (int64_t*)malloc(sizeof(int64_t) * (size_t)T);
  memcpy(phys, weights_offsets, sizeof(int64_t) * (size_t)T);
  qsort(phys, (size_t)T, sizeof(int64_t), cmp_i64);
  int32_t nphys = 0;
  for (int32_t i = 0; i < T; ++i)
    if (i == 0 || phys[i] != phys[i - 1]) phys[nphys++] = phys[i];

  int rc = 0;
  for (int32_t t = 0; t < T && rc == 0; ++t) {
    int32_t D = D_offsets[t + 1] - D_offsets[t];
    int ty = weights_tys[t];
    int32_t D_bytes = oracle_padded_row_bytes(D, ty, (int32_t)row_alignment, 4);
    int64_t next = weights_numel;
    for (int32_t i = 0; i < nphys; ++i)
      if (phys[i] > weights_offsets[t]) { next = phys[i]; break; }
    int64_t num_rows = (next - weights_offsets[t]) / D_bytes;
    int64_t o0 = read_index(offsets, idx64, (int64_t)t * B);
    int64_t o1 = read_index(offsets, idx64, (int64_t)(t + 1) * B);
    int64_t index_size = o1 - o0;
    int64_t isz = idx64 ? 8 : 4;
    int64_t elem = ty == ST_FP32 ? 4 : (ty == ST_FP16 ? 2 : 1);
    int ok = oracle_embedding_spmdm(
        ty, D, B, index_size, num_rows, dev_weights + weights_offsets[t],
        (const uint8_t*)indices + o0 * isz, idx64,
        (const uint8_t*)offsets + (int64_t)t * B * isz, idx64,
        indice_weights ? indice_weights + o0 : NULL, pooling_mode == 1,
        (uint8_t*)output + (size_t)D_offsets[t] * esz, out_ty, 0, 1, total_D,
        D_bytes / elem, 0, NULL);
    if (!ok) rc = 1 + t;
  }
  free(phys);
  return rc;
}

/* ---- array forms of the conversions, for exhaustive tests --------------- */
void oracle_half2float_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_half2float(in[i]);
}
void oracle_float2half_rn_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_float2half_rn(in[i]);
}
void oracle_float2bf16_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_float2bf16(in[i]);
}

/* ---- 8-bit float rows (hfp8) ------------------------------------------------
 * Float8ToFloat_ref (src/RefImplementations.cc:184-214): the 7 low bits go to
 * fp32's exponent / mantissa fields, the value is multiplied by
 * 2^(127 - exponent_bias), the sign bit is ORed back in. */
float oracle_float8_to_float(uint8_t input, int exponent_bits, int exponent_bias) {
  union { uint32_t i; float f; } val, mult;
  const uint32_t sign = ((uint32_t)input & 0x80u) << 24;
  val.i = ((uint32_t)input & 0x7fu) << (24 - (8 - exponent_bits));
  mult.i = (uint32_t)(127 + (127 - exponent_bias)) << 23;
  val.f *= mult.f;
  val.i |= sign;
  return val.f;
}

/* EmbeddingSpMDMFP8_ref (src/RefImplementations.cc:1544-1616): buf[j] =
 * fma(w, value(row[j]), buf[j]); no scale/bias; mean and output conversion as
 * the other kernels. skip_minus_one = 0 is the reference (an index of -1 is
 * out of range); 1 models the table-batched operator, which skips pruned rows
 * for every row type. Returns 1, or 0 where the reference returns false. */
int oracle_embedding_spmdm_fp8(
    int64_t block_size, int64_t output_size, int64_t index_size, int64_t data_size, const uint8_t* input,
    const void* indices, int idx64, const void* offsets_or_lengths, int off64, const float* weights,
    int normalize_by_lengths, void* out, int out_ty, int is_weight_positional, int use_offsets,
    int64_t output_stride, int64_t input_stride, int exponent_bits, int exponent_bias, int skip_minus_one) {
  if (output_stride == -1) output_stride = block_size;
  if (input_stride == -1) input_stride = block_size;
  float* buf = (float*)malloc(sizeof(float) * (size_t)(block_size > 0 ? block_size : 1));
  int64_t current = 0;
  int ok = 1;
  for (int64_t m = 0; m < output_size && ok; ++m) {
    memset(buf, 0, sizeof(float) * (size_t)block_size);
    const int64_t o0 = off64 ? ((const int64_t*)offsets_or_lengths)[m] : ((const int32_t*)offsets_or_lengths)[m];
    int len;
    if (use_offsets) {
      const int64_t o1 = off64 ? ((const int64_t*)offsets_or_lengths)[m + 1] : ((const int32_t*)offsets_or_lengths)[m + 1];
      len = (int)(o1 - o0);
    } else {
      len = (int)o0;
    }
    if (current + len > index_size) { ok = 0; break; }
    for (int i = 0; i < len; ++i) {
      const int64_t idx = idx64 ? ((const int64_t*)indices)[current] : ((const int32_t*)indices)[current];
      if (skip_minus_one && idx == -1) { ++current; continue; }
      if (idx < 0 || idx >= data_size) { ok = 0; break; }
      float w = 1.0f;
      if (weights) w = weights[is_weight_positional ? i : current];
      for (int64_t j = 0; j < block_size; ++j)
        buf[j] = fmaf(w, oracle_float8_to_float(input[input_stride * idx + j], exponent_bits, exponent_bias), buf[j]);
      ++current;
    }
    if (!ok) break;
    if (normalize_by_lengths && len) {
      const float scale = 1.0f / (float)len;
      for (int64_t j = 0; j < block_size; ++j) buf[j] *= scale;
    }
    for (int64_t j = 0; j < block_size; ++j) {
      const int64_t o = m * output_stride + j;
      if (out_ty == ST_FP32) ((float*)out)[o] = buf[j];
      else if (out_ty == ST_BF16) ((uint16_t*)out)[o] = oracle_float2bf16(buf[j]);
      else ((uint16_t*)out)[o] = oracle_float2half_rn(buf[j]);
    }
  }
  free(buf);
  return ok && current == index_size;
}

/* ---- no_bag (one output row per index) of the single-table kernels -------
 * EmbeddingSpMDM_ref with no_bag (src/RefImplementations.cc:1235-1288 8-bit
 * rows, :1352-1376 fp16 / bf16 / fp32 rows) and EmbeddingSpMDMNBit_ref with
 * no_bag (:1466-1484). output_size indices, no offsets:
 *   8-bit rows, 8-bit output (out_ty == ST_INT8): the first
 *     min(output_stride, input_stride) bytes of the row are copied, output
 *     rows are output_stride bytes apart;
 *   8-bit rows, float output: out[j] = convert(fma(w*scale, q[j], 0 + w*bias));
 *   plain rows: out[j] = convert(fma(w, x[j], 0));
 *   4-bit rows (out_ty == ST_INT4, the only combination the reference has):
 *     input_stride bytes are copied and output rows are input_stride apart.
 *     The reference lets idx == data_size through there (`idx > data_size`,
 *     :1478); this restatement keeps that, tests stay away from it.
 * An index of -1 is out of range in this mode whatever the layout.
 * Returns 1, or 0 where the reference returns false. */
int oracle_embedding_spmdm_nobag(
    int in_ty, int64_t block_size, int64_t output_size, int64_t data_size, const void* input, const void* indices,
    int idx64, const float* weights, void* out, int out_ty, int64_t output_stride, int64_t input_stride,
    int scale_bias_last) {
  const uint8_t* in8 = (const uint8_t*)input;
  if (output_stride == -1) output_stride = block_size;
  if (in_ty == ST_INT4 || in_ty == ST_INT2) {
    if (in_ty != ST_INT4 || out_ty != ST_INT4) return 0;
    if (input_stride == -1) input_stride = (block_size + 1) / 2 + 4;
    uint8_t* o = (uint8_t*)out;
    for (int64_t i = 0; i < output_size; ++i) {
      const int64_t idx = read_index(indices, idx64, i);
      if (idx < 0 || idx > data_size) return 0;
      memcpy(o, in8 + input_stride * idx, (size_t)input_stride);
      o += input_stride;
    }
    return 1;
  }
  if (in_ty == ST_INT8) {
    const int64_t sb = scale_bias_last ? 8 : 4;
    if (input_stride == -1) input_stride = block_size + sb;
    for (int64_t m = 0; m < output_size; ++m) {
      const int64_t idx = read_index(indices, idx64, m);
      if (idx < 0 || idx >= data_size) return 0;
      const uint8_t* row = in8 + input_stride * idx;
      if (out_ty == ST_INT8) {
        const int64_t w = output_stride < input_stride ? output_stride : input_stride;
        memcpy((uint8_t*)out + m * output_stride, row, (size_t)w);
        continue;
      }
      float weight = 1.0f;
      if (weights) weight = weights[m];
      float scale, bias;
      if (scale_bias_last) {
        float f[2];
        memcpy(f, row + block_size, 8);
        scale = weight * f[0];
        bias = weight * f[1];
      } else {
        uint16_t h[2];
        memcpy(h, row, 4);
        scale = weight * oracle_half2float(h[0]);
        bias = weight * oracle_half2float(h[1]);
      }
      const uint8_t* q = row + (scale_bias_last ? 0 : 4);
      for (int64_t j = 0; j < block_size; ++j)
        store_out(out, out_ty, m * output_stride + j, fmaf(scale, (float)q[j], 0.0f + bias));
    }
    return 1;
  }
  if (input_stride == -1) input_stride = block_size;
  for (int64_t m = 0; m < output_size; ++m) {
    const int64_t idx = read_index(indices, idx64, m);
    if (idx < 0 || idx >= data_size) return 0;
    float w = 1.0f;
    if (weights) w = weights[m];
    for (int64_t j = 0; j < block_size; ++j) {
      float x;
      if (in_ty == ST_FP32) x = ((const float*)input)[input_stride * idx + j];
      else {
        const uint16_t u = ((const uint16_t*)input)[input_stride * idx + j];
        x = in_ty == ST_BF16 ? oracle_bf162float(u) : oracle_half2float(u);
      }
      store_out(out, out_ty, m * output_stride + j, fmaf(w, x, 0.0f));
    }
  }
  return 1;
}
