// Device helpers shared by the lookup kernels: bit casts, the per-row
// accumulate of every row type, loads, output writers, error reporting.
#pragma once
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct __attribute__((packed, aligned(4))) Dwordx4 { uint32_t v[4]; };
struct __attribute__((packed, aligned(4))) Dwordx2 { uint32_t v[2]; };
struct __attribute__((packed, aligned(1))) Bytes8 { uint8_t v[8]; };
struct __attribute__((packed, aligned(1))) Bytes4 { uint8_t v[4]; };
struct __attribute__((packed, aligned(2))) Half1 { uint16_t v; };

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// A 16-bit pattern whose exponent field is zero is the half-precision
// denormal m * 2^-24. Converting it to fp32 is exact, which turns "mask a
// field of a packed word" into "have that small integer as a float" without a
// separate integer-to-float conversion; the 2^24 is folded into the row scale.
__device__ __forceinline__ float half_lo(uint32_t u) {
  return (float)__builtin_bit_cast(f16x2, u).x;
}
__device__ __forceinline__ float half_hi(uint32_t u) {
  return (float)__builtin_bit_cast(f16x2, u).y;
}

__device__ __forceinline__ constexpr int type_bits(int ty) {
  return ty == ST_FP32 ? 32 : (ty == ST_FP16 || ty == ST_BF16) ? 16 : (ty == ST_INT8 || ty == ST_FP8) ? 8 : ty == ST_INT4 ? 4 : 2;
}

__device__ __forceinline__ void report(Status* st, int32_t bit) {
  atomicOr(&st->bits, bit);
}
__device__ __forceinline__ void report_index(Status* st, int64_t pos) {
  atomicOr(&st->bits, ERR_INDEX_OUT_OF_RANGE);
  atomicMin(&st->first_bad_pos, (unsigned long long)pos);
}

// ---- per-row accumulate ---------------------------------------------------
//
// raw[] holds the VB bytes this lane loaded (VB < 4: in the low bits of raw[0]).
// fast() may pre-scale the row scale by 2^24, which is exact unless it
// overflows: the caller uses it only when |scale| < 2^100 and slow() (plain
// integer -> float conversion) otherwise. Both round identically.

template <int TY, int VB>
struct Accum;

// 8-bit rows. Two bytes of a word are spread into the two halves of a register
// with one byte permute; each half is then the half-precision denormal
// q * 2^-24, which the fma widens exactly.
template <int VB>
struct Accum<ST_INT8, VB> {
  static constexpr int E = VB;
  static constexpr bool kPrescaled = VB >= 4;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
    if constexpr (kPrescaled) {
      const float s24 = scale * 0x1p24f;
#pragma unroll
      for (int w = 0; w < VB / 4; ++w) {
        const uint32_t lo = __builtin_amdgcn_perm(0u, raw[w], 0x0c010c00u); // bytes 0, 1
        const uint32_t hi = __builtin_amdgcn_perm(0u, raw[w], 0x0c030c02u); // bytes 2, 3
        float* c = acc + 4 * w;
        c[0] = __builtin_fmaf(s24, half_lo(lo), c[0] + bias);
        c[1] = __builtin_fmaf(s24, half_hi(lo), c[1] + bias);
        c[2] = __builtin_fmaf(s24, half_lo(hi), c[2] + bias);
        c[3] = __builtin_fmaf(s24, half_hi(hi), c[3] + bias);
      }
    } else {
      slow(acc, raw, scale, bias);
    }
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t q = (raw[e / 4] >> (8 * (e % 4))) & 0xffu;
      acc[e] = __builtin_fmaf(scale, (float)q, acc[e] + bias);
    }
  }
};

// 4-bit rows. Masks leave nibbles k and k + 4 of a word in the two halves of
// a register as half-precision denormals (times 16 for the odd ones); the
// powers of two are folded into two pre-scaled copies of the row scale.
template <int VB>
struct Accum<ST_INT4, VB> {
  static constexpr int E = VB * 2;
  static constexpr bool kPrescaled = VB >= 4;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
    if constexpr (kPrescaled) {
      const float s24 = scale * 0x1p24f;
      const float s20 = scale * 0x1p20f;
#pragma unroll
      for (int w = 0; w < VB / 4; ++w) {
        const uint32_t x = raw[w];
        const uint32_t y = x >> 8;
        const uint32_t a0 = x & 0x000f000fu; // nibbles 0, 4
        const uint32_t a1 = x & 0x00f000f0u; // nibbles 1, 5 (times 16)
        const uint32_t a2 = y & 0x000f000fu; // nibbles 2, 6
        const uint32_t a3 = y & 0x00f000f0u; // nibbles 3, 7 (times 16)
        float* c = acc + 8 * w;
        c[0] = __builtin_fmaf(s24, half_lo(a0), c[0] + bias);
        c[1] = __builtin_fmaf(s20, half_lo(a1), c[1] + bias);
        c[2] = __builtin_fmaf(s24, half_lo(a2), c[2] + bias);
        c[3] = __builtin_fmaf(s20, half_lo(a3), c[3] + bias);
        c[4] = __builtin_fmaf(s24, half_hi(a0), c[4] + bias);
        c[5] = __builtin_fmaf(s20, half_hi(a1), c[5] + bias);
        c[6] = __builtin_fmaf(s24, half_hi(a2), c[6] + bias);
        c[7] = __builtin_fmaf(s20, half_hi(a3), c[7] + bias);
      }
    } else {
      slow(acc, raw, scale, bias);
    }
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t q = (raw[e / 8] >> (4 * (e % 8))) & 0xfu;
      acc[e] = __builtin_fmaf(scale, (float)q, acc[e] + bias);
    }
  }
};

template <int VB>
struct Accum<ST_INT2, VB> {
  static constexpr int E = VB * 4;
  static constexpr bool kPrescaled = false;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t q = (raw[e / 16] >> (2 * (e % 16))) & 0x3u;
      acc[e] = __builtin_fmaf(scale, (float)q, acc[e] + bias);
    }
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float a, float b) { fast(acc, raw, a, b); }
};

template <int VB>
struct Accum<ST_FP16, VB> {
  static constexpr int E = VB / 2;
  static constexpr bool kPrescaled = false;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float x = (e & 1) ? half_hi(raw[e / 2]) : half_lo(raw[e / 2]);
      acc[e] = __builtin_fmaf(w, x, acc[e]);
    }
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float a, float b) { fast(acc, raw, a, b); }
};

template <int VB>
struct Accum<ST_BF16, VB> {
  static constexpr int E = VB / 2;
  static constexpr bool kPrescaled = false;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t u = (e & 1) ? (raw[e / 2] & 0xffff0000u) : (raw[e / 2] << 16);
      acc[e] = __builtin_fmaf(w, bits_to_float(u), acc[e]);
    }
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float a, float b) { fast(acc, raw, a, b); }
};

// 8-bit floats: the 7 low bits are moved to fp32's exponent and mantissa
// fields, the value is scaled by 2^(127 - bias) and the sign bit is put back
// (Float8ToFloat_ref, src/RefImplementations.cc:184-214); then acc = fma(w, x, acc).
// `shift` and `mult` come with the call (they are the same for all lanes).
template <int VB>
struct Accum<ST_FP8, VB> {
  static constexpr int E = VB;
  static constexpr bool kPrescaled = false;
  __device__ __forceinline__ static void fp8(float (&acc)[E], const uint32_t* raw, float w, int shift, float mult) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t b = (raw[e / 4] >> (8 * (e % 4))) & 0xffu;
      const float mag = bits_to_float((b & 0x7fu) << shift) * mult;
      const float x = bits_to_float(float_to_bits(mag) | ((b & 0x80u) << 24));
      acc[e] = __builtin_fmaf(w, x, acc[e]);
    }
  }
  __device__ __forceinline__ static void fast(float (&)[E], const uint32_t*, float, float) {}
  __device__ __forceinline__ static void slow(float (&)[E], const uint32_t*, float, float) {}
};

template <int VB>
struct Accum<ST_FP32, VB> {
  static constexpr int E = VB / 4;
  static constexpr bool kPrescaled = false;
  __device__ __forceinline__ static void fast(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = __builtin_fmaf(w, bits_to_float(raw[e]), acc[e]);
  }
  __device__ __forceinline__ static void slow(float (&acc)[E], const uint32_t* raw, float a, float b) { fast(acc, raw, a, b); }
};

// ---- loads ----------------------------------------------------------------

template <int VB>
__device__ __forceinline__ void load_raw(uint32_t (&raw)[(VB + 3) / 4], const uint8_t* p) {
  if constexpr (VB == 16) {
    const Dwordx4 v = *reinterpret_cast<const Dwordx4*>(p);
    raw[0] = v.v[0]; raw[1] = v.v[1]; raw[2] = v.v[2]; raw[3] = v.v[3];
  } else if constexpr (VB == 8) {
    const Dwordx2 v = *reinterpret_cast<const Dwordx2*>(p);
    raw[0] = v.v[0]; raw[1] = v.v[1];
  } else if constexpr (VB == 4) {
    raw[0] = *reinterpret_cast<const uint32_t*>(p);
  } else if constexpr (VB == 2) {
    raw[0] = reinterpret_cast<const Half1*>(p)->v;
  } else {
    raw[0] = *p;
  }
}

// (scale, bias) of a quantised row, widened to fp32. `aligned` promises a
// 4-byte aligned address.
__device__ __forceinline__ void load_scale_bias(const uint8_t* p, bool fp32_pair, bool aligned, float& s, float& b) {
  if (fp32_pair) {
    uint32_t u0, u1;
    if (aligned) {
      const Dwordx2 v = *reinterpret_cast<const Dwordx2*>(p);
      u0 = v.v[0]; u1 = v.v[1];
    } else {
      const Bytes8 v = *reinterpret_cast<const Bytes8*>(p);
      u0 = v.v[0] | (v.v[1] << 8) | (v.v[2] << 16) | ((uint32_t)v.v[3] << 24);
      u1 = v.v[4] | (v.v[5] << 8) | (v.v[6] << 16) | ((uint32_t)v.v[7] << 24);
    }
    s = bits_to_float(u0);
    b = bits_to_float(u1);
  } else {
    uint32_t u;
    if (aligned) {
      u = *reinterpret_cast<const uint32_t*>(p);
    } else {
      const Bytes4 v = *reinterpret_cast<const Bytes4*>(p);
      u = v.v[0] | (v.v[1] << 8) | (v.v[2] << 16) | ((uint32_t)v.v[3] << 24);
    }
    s = half_lo(u);
    b = half_hi(u);
  }
}

// ---- output ---------------------------------------------------------------

__device__ __forceinline__ uint32_t to_half_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f); // round to nearest even
}
// the reference's bf16 writer: add 0x8000 to the pattern, keep the top half
// (include/fbgemm/FloatConversion.h:312-315)
__device__ __forceinline__ uint32_t to_bf16_bits(float f) { return (float_to_bits(f) + 0x8000u) >> 16; }
// two outputs in one word: bytes 2, 3 of each rounded-up pattern, picked by one byte permute
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_amdgcn_perm(float_to_bits(hi) + 0x8000u, float_to_bits(lo) + 0x8000u, 0x07060302u);
}
__device__ __forceinline__ uint32_t pack_half2(float lo, float hi) { return to_half_bits(lo) | (to_half_bits(hi) << 16); }

template <int NBYTES>
__device__ __forceinline__ void store_words(void* p, const uint32_t* w) {
  if constexpr (NBYTES >= 16) {
#pragma unroll
    for (int i = 0; i < NBYTES / 16; ++i) {
      uint4 v = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
      reinterpret_cast<uint4*>(p)[i] = v;
    }
  } else if constexpr (NBYTES == 8) {
    *reinterpret_cast<uint2*>(p) = make_uint2(w[0], w[1]);
  } else if constexpr (NBYTES == 4) {
    *reinterpret_cast<uint32_t*>(p) = w[0];
  } else {
    *reinterpret_cast<uint16_t*>(p) = (uint16_t)w[0];
  }
}

template <int E>
__device__ __forceinline__ void write_out(const LookupArgs& a, const float (&acc)[E], int64_t elem_pos, int col0, int D, bool vec_ok) {
  if (a.out_ty == ST_FP32) {
    float* o = reinterpret_cast<float*>(a.out) + elem_pos;
    if (vec_ok) {
      uint32_t w[E];
#pragma unroll
      for (int e = 0; e < E; ++e) w[e] = float_to_bits(acc[e]);
      store_words<E * 4>(o, w);
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (col0 + e < D) o[e] = acc[e];
    }
  } else {
    uint16_t* o = reinterpret_cast<uint16_t*>(a.out) + elem_pos;
    const bool bf = a.out_ty == ST_BF16;
    if (vec_ok && E >= 2) {
      uint32_t w[(E + 1) / 2];
      if (bf) {
#pragma unroll
        for (int e = 0; e + 1 < E; e += 2) w[e / 2] = pack_bf16x2(acc[e], acc[e + 1]);
      } else {
#pragma unroll
        for (int e = 0; e + 1 < E; e += 2) w[e / 2] = pack_half2(acc[e], acc[e + 1]);
      }
      store_words<E * 2>(o, w);
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (col0 + e < D) o[e] = (uint16_t)(bf ? to_bf16_bits(acc[e]) : to_half_bits(acc[e]));
    }
  }
}

// Writer of the whole-row chunk layout: the 16-byte chunk a lane holds starts
// one dword (the row header) before a 16-byte boundary of the element data, so
// its E accumulators are 4 runs of E / 4 columns, the first of them at col0
// (negative for the chunk that holds the header: that run is not output).
template <int E>
__device__ __forceinline__ void write_out_runs(const LookupArgs& a, const float (&acc)[E], int64_t row_pos, int col0, int D, bool vec_ok) {
  constexpr int GE = E / 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int cj = col0 + j * GE;
    const bool whole = cj >= 0 && cj + GE <= D;
    if (a.out_ty == ST_FP32) {
      float* o = reinterpret_cast<float*>(a.out) + row_pos + cj;
      if (whole && vec_ok) {
        uint32_t w[GE];
#pragma unroll
        for (int e = 0; e < GE; ++e) w[e] = float_to_bits(acc[j * GE + e]);
        store_words<GE * 4>(o, w);
      } else {
#pragma unroll
        for (int e = 0; e < GE; ++e)
          if (cj + e >= 0 && cj + e < D) o[e] = acc[j * GE + e];
      }
    } else {
      uint16_t* o = reinterpret_cast<uint16_t*>(a.out) + row_pos + cj;
      const bool bf = a.out_ty == ST_BF16;
      if (whole && vec_ok) {
        uint32_t w[GE / 2];
        if (bf) {
#pragma unroll
          for (int e = 0; e < GE; e += 2) w[e / 2] = pack_bf16x2(acc[j * GE + e], acc[j * GE + e + 1]);
        } else {
#pragma unroll
          for (int e = 0; e < GE; e += 2) w[e / 2] = pack_half2(acc[j * GE + e], acc[j * GE + e + 1]);
        }
        store_words<GE * 2>(o, w);
      } else {
#pragma unroll
        for (int e = 0; e < GE; ++e)
          if (cj + e >= 0 && cj + e < D) o[e] = (uint16_t)(bf ? to_bf16_bits(acc[j * GE + e]) : to_half_bits(acc[j * GE + e]));
      }
    }
  }
}


// ---- shared by the kernels ---------------------------------------------------

__device__ __forceinline__ int64_t read_offset(const void* p, bool is64, int64_t i) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}

// What one staging lane leaves in LDS for the lanes that own the columns:
// where the row is, and what to multiply it with.
struct __attribute__((aligned(8))) StageRow {
  int64_t off; // byte offset of the row from the table's first row, or < 0: nothing to add
};
struct __attribute__((aligned(8))) StageMul {
  float scale; // w * row scale (quantised rows) or w (fp16 / bf16 / fp32 rows)
  float bias;  // w * row bias
};

constexpr int MAX_GROUPS = 32; // bags per wave at most; lanes per bag >= 2
constexpr int MAX_ROUND = 8;
constexpr int64_t NO_ENTRY = INT64_MIN;

} // namespace fbgemm_amd
