// gfx950 kernels of the quantized embedding-bag lookup: gather packed rows,
// dequantize in registers, pool in fp32 in index order, write fp32/fp16/bf16.
//
// Arithmetic contract (what the reference's CPU path computes,
// src/RefImplementations.cc:1196-1346,1428-1541): for every index of a bag,
// in order,
//     scale = w * row_scale;  bias = w * row_bias;
//     acc[j] = fma(scale, q[j], acc[j] + bias)            (quantised rows)
//     acc[j] = fma(w, x[j], acc[j])                       (fp16/bf16/fp32 rows)
// then acc *= 1.0f / len for mean pooling (len counts skipped rows) and one
// conversion to the output type. Every output column is owned by exactly one
// lane and rows are consumed in index order, so the fp32 sequence of roundings
// is the reference's and results are bit-identical, not merely close.
//
// Lane mapping: `lanes` consecutive lanes of a wave share one bag; lane `sub`
// of the group owns the `vb` bytes of every row that start at
// (pass * lanes + sub) * vb, i.e. vb * 8 / bits consecutive output columns. A
// wave therefore pools bags_per_wave(lanes) bags at once and each row is fetched with
// one coalesced run of 16-byte loads.
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

// ---- one wave, one table ----------------------------------------------------

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

// One wave pools bags_per_wave(lanes) bags of one table, `RN` entries of every bag per
// round. Each lane owns C chunks of VB bytes of every row: chunk c of lane
// `sub` starts at byte (c * lanes + sub) * VB of the row data, so every load
// instruction of the wave reads contiguous bytes of each row.
//
// Per-entry work (index load, per-sample weight, -1 / bounds / remap handling,
// row offset, the scale/bias fetch and its two products with the weight) is
// done ONCE per entry by a staging lane and handed to the `lanes` column lanes
// of the bag through LDS, instead of being repeated by each of them.
//
// The memory system charges per 128-byte line request, so a row's scale/bias
// must not cost a request of its own: the staging lane loads them in the same
// round, immediately before the column lanes load the row's data, and the two
// accesses to the row's first line merge in the L1. While the loads are in
// flight the indices of the next round are fetched.
//
// A round in which every lane of the wave has RN rows to add (the normal case
// once bags are ordered by length) runs without a single predicate.
//
// PRESCALE selects the arithmetic route of the 4- and 8-bit rows: the
// pre-scaled one (scale * 2^24 times a half-precision denormal) is exact unless
// scale * 2^24 overflows. A wave that meets |scale| >= 2^100 gives up, returns
// false, and its work is redone from the start by the PRESCALE = false
// instance, which converts integers to float the plain way.
//
// INHDR (4- and 8-bit rows whose fp16 scale/bias pair comes first and whose
// stride is a multiple of 16): the lanes of a bag own the 16-byte chunks of the
// whole row, header included, so that the header costs no memory request of
// its own: the lane that holds chunk 0 hands it to the others through a lane
// permute. `lanes` then need not divide 64; the lanes left over shadow the last
// bag of the wave (same addresses, nothing written), and so do chunk slots past
// the end of the row.
template <typename index_t, bool GENERAL, int TY, int VB, int C, int ROUND, bool PRESCALE, bool INHDR = false>
__device__ __forceinline__ bool pool_bags(const LookupArgs& a, const TableDesc& d, int table, int first_slot,
                                          int lane, StageRow* stage_row, StageMul* stage_mul) {
  constexpr int BITS = type_bits(TY);
  constexpr int E = VB * 8 / BITS;
  constexpr int NW = (VB + 3) / 4;
  constexpr bool QUANT = TY == ST_INT8 || TY == ST_INT4 || TY == ST_INT2;
  constexpr bool ALIGNED = VB >= 4;
  constexpr int MAXR = 2; // entries one staging lane handles per round, at most
  using Acc = Accum<TY, VB>;

  static_assert(!INHDR || (VB == 16 && QUANT), "whole-row chunks are 16 bytes of a quantised row");
  const int S = d.lanes;
  const int G = bags_per_wave(S, d.packed);
  // quarter q of the wave holds bags q * (16 / S) ...; its last 16 % S lanes idle
  int grp, sub;
  bool idle;
  // divisions by S through the table's reciprocal (exact for arguments up to 64)
  const uint32_t recip = (uint32_t)d.lanes_recip;
  if (S <= 16 && !d.packed) {
    const int per_q = (int)((16u * recip) >> 16);
    const int j = lane & 15;
    const int gq = (int)(((uint32_t)j * recip) >> 16);
    idle = gq >= per_q;
    grp = (lane >> 4) * per_q + (idle ? per_q - 1 : gq);
    sub = j - gq * S;
  } else {
    grp = (int)(((uint32_t)lane * recip) >> 16);
    sub = lane - grp * S;
    idle = grp >= G;
  }
  const int slot = first_slot + grp;
  const int lgrp = idle ? G - 1 : grp;  // idle lanes never enter the loops; any valid staging slot will do
  const bool bag_ok = !idle && slot < a.B;
  const bool reporter = sub == 0;
  // staging lanes per bag: a power of two <= lanes; entries per round: ROUND,
  // or what MAXR entries per staging lane allow
  const int SLmax = S >= 8 ? 8 : (S >= 4 ? 4 : 2);
  const int RN = ROUND < SLmax * MAXR ? ROUND : SLmax * MAXR;
  const int SL = SLmax < RN ? SLmax : RN;
  const int R = RN / SL;
  const bool stager = bag_ok && sub < SL;

  // Bags are taken in the order the scheduler left them (longest first), so
  // that the bags sharing a wave have nearly equal lengths. Positions are
  // counted the way the reference counts `current`: relative to the first
  // offset of the table's slice.
  int bag = slot;
  int64_t pos0 = 0;
  int64_t len = 0;
  if (bag_ok) {
    const int64_t ob = (int64_t)table * a.B;
    int64_t o0, o1;
    if (a.order) {
      const BagEntry be = a.order[ob + slot];
      bag = be.bag;
      o0 = be.o0;
      o1 = be.o1;
    } else {
      o0 = read_offset(a.offsets, a.off64, ob + bag);
      o1 = read_offset(a.offsets, a.off64, ob + bag + 1);
    }
    int64_t base = 0;
    if (GENERAL && a.check_total) base = read_offset(a.offsets, a.off64, ob);
    pos0 = o0 - base; // table-batched calls index the shared array: base = 0
    len = o1 - o0;
    if (len < 0) {
      if (reporter) report(a.status, ERR_NEGATIVE_LENGTH);
      len = 0;
    }
    if (len > 0x7fffffffLL || pos0 < 0 || pos0 + len > a.index_size) {
      if (reporter) report(a.status, ERR_BAG_OVERRUN);
      len = 0;
    }
    if (GENERAL && a.check_total && bag == a.B - 1 && o1 - base != a.index_size && reporter)
      report(a.status, ERR_LENGTH_MISMATCH);
  }
  const int n = (int)len; // same for every lane of the bag

  // pruned tables: logical ids go through the table's slice of the remap array
  int64_t remap_base = 0, remap_cap = 0;
  bool remapped = false;
  if (GENERAL && a.remap) {
    remapped = true;
    remap_cap = a.remap_rows;
    if (a.remap_offsets) {
      remap_base = a.remap_offsets[table];
      remap_cap = a.remap_offsets[table + 1] - remap_base;
      remapped = remap_cap > 0;
    }
  }

  const index_t* idx = reinterpret_cast<const index_t*>(a.indices);
  const uint8_t* wbase = (d.placement ? a.weights[1] : a.weights[0]) + d.weights_offset;
  const uint8_t* psb = wbase + d.sb_off;
  StageRow* my_row = stage_row + lgrp * RN;
  StageMul* my_mul = stage_mul + lgrp * RN;
  // the reference keeps the bag length in an int when it forms 1/len
  const float inv_len = (a.normalize && n > 0) ? 1.0f / (float)n : 1.0f;
  const int chunk_stride = S * VB; // bytes between a lane's consecutive chunks

  for (int pass = 0; pass < d.passes; ++pass) {
    const int chunk0 = pass * S * C + sub;
    bool on[C];
    bool all_on = bag_ok;
    int rowb[C]; // INHDR: byte offset of the lane's chunks inside the row
    if constexpr (INHDR) {
      const int nchunks = (d.data_bytes + 4 + VB - 1) / VB;
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const int k = chunk0 + c * S;
        on[c] = bag_ok && k < nchunks;
        rowb[c] = (k < nchunks ? k : nchunks - 1) * VB; // a slot past the row shadows the last chunk
      }
    } else {
#pragma unroll
      for (int c = 0; c < C; ++c) {
        on[c] = bag_ok && (chunk0 + c * S) * VB < d.data_bytes;
        all_on = all_on && on[c];
        rowb[c] = 0;
      }
    }
    const uint8_t* pdata = INHDR ? wbase : wbase + d.data_off + chunk0 * VB;

    float acc[C][E];
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
      for (int e = 0; e < E; ++e) acc[c][e] = 0.0f;

    // registers of the staging lanes
    int64_t nrow[MAXR]; // raw index of the next round (loads in flight)
    float nw[MAXR];
    int64_t coff[MAXR]; // row offset and weight of the round being pooled
    float cw[MAXR];

    auto load_idx = [&](int round) {
#pragma unroll
      for (int rr = 0; rr < MAXR; ++rr) {
        nrow[rr] = NO_ENTRY;
        nw[rr] = 1.0f;
        const int i = round * RN + sub + rr * SL;
        if (rr < R && stager && i < n) {
          nrow[rr] = (int64_t)idx[pos0 + i];
          if (a.sample_weights) nw[rr] = a.sample_weights[(GENERAL && a.positional) ? (int64_t)i : pos0 + i];
        }
      }
    };
    // index -> row offset, or "nothing to add"; publish the offsets of `round`.
    // Returns true on a staging lane that leaves a hole (no entry, or a
    // skipped / rejected one) in the round.
    auto stage_rows = [&](int round) -> bool {
      bool hole = false;
#pragma unroll
      for (int rr = 0; rr < MAXR; ++rr) {
        int64_t row = nrow[rr];
        int64_t off = -1;
        if (rr < R && row != NO_ENTRY) {
          const int64_t pos = pos0 + round * RN + sub + rr * SL;
          bool ok = true;
          if (GENERAL && remapped) {
            if (row < 0 || row >= remap_cap) {
              if (pass == 0) report_index(a.status, pos);
              ok = false;
            } else {
              row = a.remap64 ? reinterpret_cast<const int64_t*>(a.remap)[remap_base + row]
                              : (int64_t) reinterpret_cast<const int32_t*>(a.remap)[remap_base + row];
              ok = row != -1;
              if (ok && (row < 0 || row >= d.num_rows)) {
                if (pass == 0) report_index(a.status, pos);
                ok = false;
              }
            }
          } else if (d.skip_minus_one && row == -1) {
            ok = false;
          } else if (row < 0 || row >= d.num_rows) {
            if (pass == 0) report_index(a.status, pos);
            ok = false;
          }
          if (ok) off = row * d.row_stride;
        }
        coff[rr] = off;
        cw[rr] = nw[rr];
        if (rr < R && stager) {
          hole = hole || (off < 0 && round * RN < n); // a bag that has ended leaves the loop instead
          my_row[sub + rr * SL].off = off;
          // Plain rows: the multiplier is the weight. A hole gets (-0, -0),
          // which leaves every accumulator exactly as it is:
          // fma(-0, q, acc + -0) == acc for any acc, +0 and -0 included.
          if (!QUANT || INHDR || off < 0) {
            StageMul m;
            m.scale = off < 0 ? -0.0f : nw[rr];
            m.bias = -0.0f;
            my_mul[sub + rr * SL] = m;
          }
        }
      }
      return hole;
    };

    // wave-uniform: every lane of the wave pools a bag and owns C live chunks
    // (whole-row chunks: slots past the row are clamped, lanes without a bag never enter the loop)
    const bool wave_on = INHDR || (__builtin_amdgcn_ballot_w64(!all_on) == 0ull && __builtin_amdgcn_ballot_w64(true) == ~0ull);
    load_idx(0);
    // wave-uniform: the staged round has RN rows to add for every bag of the wave
    // (the staging call comes first on its own line: it must run on every wave)
    const bool hole0 = stage_rows(0);
    bool fast = wave_on && __builtin_amdgcn_ballot_w64(hole0) == 0ull;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    bool give_up = false;
    for (int r = 0; r * RN < n; ++r) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      uint32_t raw[ROUND][C][NW];
      uint32_t h0[MAXR], h1[MAXR];
      const int left = min(n - r * RN, RN);
      // scale/bias first, so that their wait does not cover the row loads
      if constexpr (QUANT && !INHDR) {
#pragma unroll
        for (int rr = 0; rr < MAXR; ++rr) {
          if (rr < R && stager && coff[rr] >= 0) {
            const uint8_t* p = psb + coff[rr];
            if (d.sb_fp32) {
              if constexpr (ALIGNED) {
                const Dwordx2 v = *reinterpret_cast<const Dwordx2*>(p);
                h0[rr] = v.v[0]; h1[rr] = v.v[1];
              } else {
                const Bytes8 v = *reinterpret_cast<const Bytes8*>(p);
                h0[rr] = v.v[0] | (v.v[1] << 8) | (v.v[2] << 16) | ((uint32_t)v.v[3] << 24);
                h1[rr] = v.v[4] | (v.v[5] << 8) | (v.v[6] << 16) | ((uint32_t)v.v[7] << 24);
              }
            } else {
              if constexpr (ALIGNED) {
                h0[rr] = *reinterpret_cast<const uint32_t*>(p);
              } else {
                const Bytes4 v = *reinterpret_cast<const Bytes4*>(p);
                h0[rr] = v.v[0] | (v.v[1] << 8) | (v.v[2] << 16) | ((uint32_t)v.v[3] << 24);
              }
            }
          }
        }
      }
      if (fast) {
#pragma unroll
        for (int e = 0; e < ROUND; ++e) {
          if (e < RN) {
            const uint8_t* p = pdata + my_row[e].off;
#pragma unroll
            for (int c = 0; c < C; ++c) load_raw<VB>(raw[e][c], INHDR ? p + rowb[c] : p + c * chunk_stride);
          }
        }
      } else {
        // ragged round: rows that are not there read as zeros and are
        // multiplied by -0 below
#pragma unroll
        for (int e = 0; e < ROUND; ++e) {
          if (e < RN && __builtin_amdgcn_ballot_w64(e < left) != 0ull) {
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
              for (int w = 0; w < NW; ++w) raw[e][c][w] = 0u;
            if (e < left) {
              const int64_t off = my_row[e].off;
              if (off >= 0) {
#pragma unroll
                for (int c = 0; c < C; ++c) {
                  if constexpr (INHDR) load_raw<VB>(raw[e][c], pdata + off + rowb[c]);
                  else if (on[c]) load_raw<VB>(raw[e][c], pdata + off + c * chunk_stride);
                }
              }
            }
          }
        }
      }
      load_idx(r + 1);
      if constexpr (QUANT && !INHDR) {
        bool big = false;
#pragma unroll
        for (int rr = 0; rr < MAXR; ++rr) {
          if (rr < R && stager && coff[rr] >= 0) {
            const float rs = d.sb_fp32 ? bits_to_float(h0[rr]) : half_lo(h0[rr]);
            const float rb = d.sb_fp32 ? bits_to_float(h1[rr]) : half_hi(h0[rr]);
            StageMul m;
            m.scale = cw[rr] * rs;
            m.bias = cw[rr] * rb;
            big = big || !(__builtin_fabsf(m.scale) < 0x1p100f);
            my_mul[sub + rr * SL] = m;
          }
        }
        if constexpr (PRESCALE && Acc::kPrescaled) {
          if (__builtin_amdgcn_ballot_w64(big) != 0ull) {
            give_up = true;
            break;
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      // One straight-line accumulate for the whole wave; lanes past the end of
      // their bag add holes.
      bool big = false;
#pragma unroll
      for (int e = 0; e < ROUND; ++e) {
        if (e < RN && (fast || __builtin_amdgcn_ballot_w64(e < left) != 0ull)) {
          StageMul m = my_mul[e];
          if constexpr (INHDR) {
            // the row header sits in the first dword of chunk 0, which the first
            // lane of the group holds (zeros for a row that is not there)
            const uint32_t h = (uint32_t)__builtin_amdgcn_ds_bpermute((lane - sub) * 4, (int)raw[e][0][0]);
            m.bias = m.scale * half_hi(h);
            m.scale = m.scale * half_lo(h);
            big = big || !(__builtin_fabsf(m.scale) < 0x1p100f);
          }
#pragma unroll
          for (int c = 0; c < C; ++c) {
            if constexpr (TY == ST_FP8) Acc::fp8(acc[c], raw[e][c], m.scale, a.fp8_shift, a.fp8_mult);
            else if constexpr (PRESCALE) Acc::fast(acc[c], raw[e][c], m.scale, m.bias);
            else Acc::slow(acc[c], raw[e][c], m.scale, m.bias);
          }
        }
      }
      if constexpr (INHDR && PRESCALE && Acc::kPrescaled) {
        if (__builtin_amdgcn_ballot_w64(big) != 0ull) {
          give_up = true;
          break;
        }
      }
      __builtin_amdgcn_wave_barrier();
      // offsets (and plain weights) of the next round; the column lanes have
      // read this round's entries by now
      const bool hole = stage_rows(r + 1);
      fast = wave_on && __builtin_amdgcn_ballot_w64(hole) == 0ull;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }

    if (__builtin_amdgcn_ballot_w64(give_up) != 0ull) return false; // every lane of the wave is back here

    const bool vec_ok = a.out_aligned && ((d.vec_store >> (a.out_ty == ST_FP32 ? 0 : 1)) & 1);
#pragma unroll
    for (int c = 0; c < C; ++c) {
      if (on[c]) {
        if (a.normalize && n > 0) {
#pragma unroll
          for (int e = 0; e < E; ++e) acc[c][e] *= inv_len;
        }
        if constexpr (INHDR) {
          const int col0 = (chunk0 + c * S) * E - E / 4;
          write_out_runs<E>(a, acc[c], (int64_t)bag * a.out_stride + d.out_col, col0, d.D, vec_ok);
        } else {
          const int col0 = (chunk0 + c * S) * E;
          const int64_t elem_pos = (int64_t)bag * a.out_stride + d.out_col + col0;
          write_out<E>(a, acc[c], elem_pos, col0, d.D, vec_ok);
        }
      }
    }
  }
  return true;
}

template <typename index_t, bool GENERAL, int TY, int VB, int C, int ROUND, bool INHDR = false>
__device__ __forceinline__ void run_bags(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane,
                                         StageRow* stage_row, StageMul* stage_mul) {
  if constexpr (Accum<TY, VB>::kPrescaled) {
    if (!pool_bags<index_t, GENERAL, TY, VB, C, ROUND, true, INHDR>(a, d, table, first_slot, lane, stage_row, stage_mul))
      pool_bags<index_t, GENERAL, TY, VB, C, ROUND, false, INHDR>(a, d, table, first_slot, lane, stage_row, stage_mul);
  } else {
    pool_bags<index_t, GENERAL, TY, VB, C, ROUND, true, INHDR>(a, d, table, first_slot, lane, stage_row, stage_mul);
  }
}

// Row types and the lane shapes the host may pick for them (TableDesc::vb,
// TableDesc::chunks): 16-byte chunks with up to 4 (fp16 / bf16 / fp32), 2
// (int8) or 1 (int4) chunks per lane so that a lane holds at most 32
// accumulators; 4-byte and element-sized chunks for everything else.
template <typename index_t, bool GENERAL, int TY>
__device__ __forceinline__ void pool_dispatch_vb(const LookupArgs& a, const TableDesc& d, int table, int first_slot,
                                                 int lane, StageRow* stage_row, StageMul* stage_mul) {
  constexpr int BITS = type_bits(TY);
  constexpr int MINVB = BITS >= 16 ? BITS / 8 : 1;
  constexpr int MAXC = BITS >= 16 ? 4 : (BITS == 8 ? 2 : 1);
  // rows in flight per lane: ROUND * chunks = 8 loads of 16 bytes
  if constexpr (TY == ST_INT4 || TY == ST_INT8) {
    if (d.inline_hdr) {
      if (d.chunks == 2 && MAXC >= 2) run_bags<index_t, GENERAL, TY, 16, (MAXC >= 2 ? 2 : 1), 4, true>(a, d, table, first_slot, lane, stage_row, stage_mul);
      else run_bags<index_t, GENERAL, TY, 16, 1, 8, true>(a, d, table, first_slot, lane, stage_row, stage_mul);
      return;
    }
  }
  if (d.vb == 16) {
    if constexpr (TY == ST_INT2) {
      run_bags<index_t, GENERAL, TY, 4, 1, 8>(a, d, table, first_slot, lane, stage_row, stage_mul); // not selected by the host
    } else {
      if (d.chunks == 4 && MAXC >= 4) run_bags<index_t, GENERAL, TY, 16, (MAXC >= 4 ? 4 : 1), 2>(a, d, table, first_slot, lane, stage_row, stage_mul);
      else if (d.chunks == 2 && MAXC >= 2) run_bags<index_t, GENERAL, TY, 16, (MAXC >= 2 ? 2 : 1), 4>(a, d, table, first_slot, lane, stage_row, stage_mul);
      else run_bags<index_t, GENERAL, TY, 16, 1, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
    }
  } else if (d.vb == 4) {
    run_bags<index_t, GENERAL, TY, 4, 1, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
  } else {
    run_bags<index_t, GENERAL, TY, MINVB, 1, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
  }
}

#ifndef FBGEMM_AMD_MIN_WAVES
#define FBGEMM_AMD_MIN_WAVES 3 // waves per SIMD the register allocation must leave room for
#endif

// One item of the work list: `wave` is the position in the list (or the wave's
// number for a single-table call).
template <typename index_t, bool GENERAL>
__device__ __forceinline__ void run_item(const LookupArgs& a, int64_t wave, int lane, StageRow* stage_row, StageMul* stage_mul) {
  int table = 0, first_slot;
  if (a.work) {
    const WaveWork ww = a.work[wave];
    table = ww.table;
    first_slot = ww.first_bag;
  } else {
    first_slot = (int)(wave * bags_per_wave(a.single.lanes, a.single.packed));
  }
  const TableDesc d = a.tables ? a.tables[table] : a.single;
#ifdef FBGEMM_AMD_ONLY_TY // register-budget experiments: compile a single row type
  if (d.ty == FBGEMM_AMD_ONLY_TY) pool_dispatch_vb<index_t, GENERAL, FBGEMM_AMD_ONLY_TY>(a, d, table, first_slot, lane, stage_row, stage_mul);
#else
  switch (d.ty) {
    case ST_INT4: pool_dispatch_vb<index_t, GENERAL, ST_INT4>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_INT8: pool_dispatch_vb<index_t, GENERAL, ST_INT8>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_FP16: pool_dispatch_vb<index_t, GENERAL, ST_FP16>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_INT2: pool_dispatch_vb<index_t, GENERAL, ST_INT2>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_FP32: pool_dispatch_vb<index_t, GENERAL, ST_FP32>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_BF16: pool_dispatch_vb<index_t, GENERAL, ST_BF16>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_FP8: pool_dispatch_vb<index_t, GENERAL, ST_FP8>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    default: break;
  }
#endif
}

#ifdef FBGEMM_AMD_WAVE_TRACE
__device__ __forceinline__ void trace_item(const LookupArgs& a, int64_t wave, int lane, unsigned long long t0) {
  if (a.trace && lane == 0) {
    unsigned long long* t = a.trace + (size_t)wave * 4;
    const unsigned hw = __builtin_amdgcn_s_getreg((31 << 11) | 4);   // HW_ID
    const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20);  // XCC_ID
    t[0] = t0;
    t[1] = wall_clock64();
    t[2] = (unsigned long long)hw | ((unsigned long long)xcc << 32);
    t[3] = (unsigned long long)blockIdx.x | ((unsigned long long)(a.work ? a.work[wave].table : 0) << 32);
  }
}
#endif

// One wave per workgroup: waves come and go independently, and a workgroup
// needs no more than its own 4 KB of LDS.
// GENERAL = false is the table-batched operator's subset (no logical->physical
// remap, no positional weights, offsets indexing one shared index array).
//
// The work list of a table-batched call is 8 runs, one per XCD: whole tables
// (or slices of them) are pinned to one XCD's L2 instead of spreading their hot
// rows over all eight. Workgroup i takes item i >> 3 of run i & 7 (workgroups
// are handed to the XCDs round-robin).
template <typename index_t, bool GENERAL>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(FBGEMM_AMD_MIN_WAVES, 8))) void lookup_kernel(const LookupArgs a) {
  __shared__ StageRow stage_row[MAX_GROUPS * MAX_ROUND];
  __shared__ StageMul stage_mul[MAX_GROUPS * MAX_ROUND];
  const int lane = threadIdx.x;
  int64_t wave;
  if (a.xcd_start) {
    const int xb = blockIdx.x & 7;
    const int64_t w = (int64_t)(blockIdx.x >> 3);
    const int64_t lo = a.xcd_start[xb], hi = a.xcd_start[xb + 1];
    if (w >= hi - lo) return;
    wave = lo + w;
  } else {
    wave = (int64_t)blockIdx.x;
    if (wave >= a.num_waves) return;
  }
#ifdef FBGEMM_AMD_WAVE_TRACE
  const unsigned long long trace_t0 = wall_clock64();
#endif
  run_item<index_t, GENERAL>(a, wave, lane, stage_row, stage_mul);
#ifdef FBGEMM_AMD_WAVE_TRACE
  trace_item(a, wave, lane, trace_t0);
#endif
}

// ---- bag scheduler -------------------------------------------------------------
//
// One workgroup per table orders the table's bags by length, longest first
// (counting sort over lengths, lengths >= SORT_BINS - 1 share the first bin).
// Waves then take consecutive runs of the order, so the bags a wave pools side
// by side need the same number of rounds and no lane idles behind a long
// neighbour. Ties are placed in arrival order of the LDS atomics: the order
// may differ between runs, the results cannot (each bag is summed on its own).
constexpr int SORT_BINS = 1024;

__global__ __launch_bounds__(1024) void bag_order_kernel(const void* offsets, int off64, int32_t B, BagEntry* order) {
  __shared__ int bins[SORT_BINS];
  __shared__ int partial[1024];
  const int t = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t ob = (int64_t)t * B;
  for (int i = tid; i < SORT_BINS; i += 1024) bins[i] = 0;
  __syncthreads();
  // bin of a bag: SORT_BINS - 1 - min(length, SORT_BINS - 1), so that the longest come first
  // the first two bags of every thread stay in registers between the two passes
  int64_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;
  for (int b = tid, it = 0; b < B; b += 1024, ++it) {
    const int64_t o0 = read_offset(offsets, off64, ob + b), o1 = read_offset(offsets, off64, ob + b + 1);
    if (it == 0) {
      a0 = o0;
      a1 = o1;
    } else if (it == 1) {
      b0 = o0;
      b1 = o1;
    }
    int64_t len = o1 - o0;
    len = len < 0 ? 0 : (len > SORT_BINS - 1 ? SORT_BINS - 1 : len);
    atomicAdd(&bins[SORT_BINS - 1 - (int)len], 1);
  }
  __syncthreads();
  // exclusive scan of the SORT_BINS (== blockDim) counters: inside each wave
  // through lane shuffles, then over the 16 wave totals
  const int mine = bins[tid];
  int incl = mine;
  const int lane = tid & 63;
  for (int step = 1; step < 64; step <<= 1) {
    const int v = __shfl_up(incl, step, 64);
    if (lane >= step) incl += v;
  }
  if (lane == 63) partial[tid >> 6] = incl;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < (tid >> 6); ++w) before += partial[w];
  bins[tid] = before + incl - mine;
  __syncthreads();
  for (int b = tid, it = 0; b < B; b += 1024, ++it) {
    BagEntry be;
    if (it == 0) {
      be.o0 = a0;
      be.o1 = a1;
    } else if (it == 1) {
      be.o0 = b0;
      be.o1 = b1;
    } else {
      be.o0 = read_offset(offsets, off64, ob + b);
      be.o1 = read_offset(offsets, off64, ob + b + 1);
    }
    int64_t len = be.o1 - be.o0;
    len = len < 0 ? 0 : (len > SORT_BINS - 1 ? SORT_BINS - 1 : len);
    const int p = atomicAdd(&bins[SORT_BINS - 1 - (int)len], 1);
    be.bag = b;
    be.pad0 = 0;
    be.pad1 = 0;
    order[ob + p] = be;
  }
}

// ---- helpers ----------------------------------------------------------------

// lengths -> offsets (exclusive prefix sum), one workgroup. Used when the
// caller passes Caffe2-style lengths instead of offsets.
template <typename T>
__global__ __launch_bounds__(1024) void lengths_to_offsets_kernel(const T* lengths, int64_t n, int64_t* offsets) {
  __shared__ int64_t part[1024];
  const int tid = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = (int64_t)tid * per;
  const int64_t hi = lo + per < n ? lo + per : n;
  int64_t sum = 0;
  for (int64_t i = lo; i < hi; ++i) sum += (int64_t)(int)lengths[i];
  part[tid] = sum;
  __syncthreads();
  for (int step = 1; step < 1024; step <<= 1) {
    int64_t v = tid >= step ? part[tid - step] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int64_t run = part[tid] - sum;
  for (int64_t i = lo; i < hi; ++i) {
    offsets[i] = run;
    run += (int64_t)(int)lengths[i];
  }
  if (tid == 1023) offsets[n] = part[1023];
}

__global__ void status_clear_kernel(Status* st) {
  st->bits = 0;
  st->pad = 0;
  st->first_bad_pos = ~0ull;
}

// dense[i] = remap[remap_offsets[t] + idx[i]] for tables with a mapping, a copy
// otherwise (…/embedding_forward_quantized_cpu_template.cpp:605-659).
template <typename index_t, typename remap_t>
__global__ __launch_bounds__(256) void pruned_array_lookup_kernel(
    const index_t* indices, const index_t* offsets, const remap_t* remap,
    const int64_t* remap_offsets, int32_t B, int32_t T, index_t* dense) {
  const int t = blockIdx.y;
  const int64_t rs = remap_offsets[t], re = remap_offsets[t + 1];
  const int64_t is = offsets[(int64_t)t * B], ie = offsets[(int64_t)(t + 1) * B];
  const bool mapped = re - rs > 0;
  for (int64_t i = is + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ie; i += (int64_t)gridDim.x * blockDim.x) {
    index_t v = indices[i];
    // an id outside the mapping reads nothing (the reference reads out of bounds there)
    if (mapped) v = (v >= 0 && (int64_t)v < re - rs) ? (index_t)remap[rs + v] : (index_t)-1;
    dense[i] = v;
  }
}

// Plain 16-byte-per-lane copy of a known size: the yardstick hardware byte
// counters are scaled against.
__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4* src, uint4* dst, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// ---- launchers (called from the C ABI) ---------------------------------------

hipError_t launch_calibration_copy(const void* src, void* dst, int64_t bytes, hipStream_t stream) {
  const int64_t n16 = bytes / 16;
  if (n16 <= 0) return hipSuccess;
  hipLaunchKernelGGL(calibration_copy_kernel, dim3(256 * 16), dim3(256), 0, stream, (const uint4*)src, (uint4*)dst, n16);
  return hipGetLastError();
}

hipError_t launch_lookup(const LookupArgs& a, bool idx64, hipStream_t stream) {
  if (a.num_waves <= 0) return hipSuccess;
  const int64_t blocks = a.xcd_start ? 8 * a.num_waves : a.num_waves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool general = a.remap || a.positional || a.check_total;
  const dim3 grid((unsigned)blocks), block(64);
  if (general) {
    if (idx64) hipLaunchKernelGGL((lookup_kernel<int64_t, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((lookup_kernel<int32_t, true>), grid, block, 0, stream, a);
  } else {
    if (idx64) hipLaunchKernelGGL((lookup_kernel<int64_t, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((lookup_kernel<int32_t, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

hipError_t launch_bag_order(const void* offsets, bool off64, int32_t B, int32_t T, BagEntry* order, hipStream_t stream) {
  if (T <= 0 || B <= 0) return hipSuccess;
  hipLaunchKernelGGL(bag_order_kernel, dim3((unsigned)T), dim3(1024), 0, stream, offsets, off64 ? 1 : 0, B, order);
  return hipGetLastError();
}

hipError_t launch_lengths_to_offsets(const void* lengths, bool is64, int64_t n, int64_t* offsets, hipStream_t stream) {
  if (is64) hipLaunchKernelGGL(lengths_to_offsets_kernel<int64_t>, dim3(1), dim3(1024), 0, stream, (const int64_t*)lengths, n, offsets);
  else hipLaunchKernelGGL(lengths_to_offsets_kernel<int32_t>, dim3(1), dim3(1024), 0, stream, (const int32_t*)lengths, n, offsets);
  return hipGetLastError();
}

hipError_t launch_status_clear(Status* st, hipStream_t stream) {
  hipLaunchKernelGGL(status_clear_kernel, dim3(1), dim3(1), 0, stream, st);
  return hipGetLastError();
}

hipError_t launch_pruned_array_lookup(const void* indices, const void* offsets, bool idx64, const void* remap,
                                      bool remap64, const int64_t* remap_offsets, int32_t B, int32_t T,
                                      void* dense, hipStream_t stream) {
  if (T <= 0 || B <= 0) return hipSuccess;
  dim3 grid(64, (unsigned)T), block(256);
  if (idx64 && remap64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int64_t, int64_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int64_t*)remap, remap_offsets, B, T, (int64_t*)dense);
  else if (idx64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int64_t, int32_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int32_t*)remap, remap_offsets, B, T, (int64_t*)dense);
  else if (remap64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int32_t, int64_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int64_t*)remap, remap_offsets, B, T, (int32_t*)dense);
  else
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int32_t, int32_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int32_t*)remap, remap_offsets, B, T, (int32_t*)dense);
  return hipGetLastError();
}

} // namespace fbgemm_amd
