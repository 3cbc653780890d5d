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
// wave therefore pools 64 / lanes bags at once and each row is fetched with
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
  return ty == ST_FP32 ? 32 : (ty == ST_FP16 || ty == ST_BF16) ? 16 : ty == ST_INT8 ? 8 : ty == ST_INT4 ? 4 : 2;
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
// Products with |scale| >= 2^100 cannot take the pre-scaled route (scale * 2^24
// would overflow); they use plain integer->float conversion instead.

template <int TY, int VB>
struct Accum;

template <int VB>
struct Accum<ST_INT8, VB> {
  static constexpr int E = VB;
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t q = (raw[e / 4] >> (8 * (e % 4))) & 0xffu;
      acc[e] = __builtin_fmaf(scale, (float)q, acc[e] + bias);
    }
  }
};

template <int VB>
struct Accum<ST_INT4, VB> {
  static constexpr int E = VB * 2;
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
    if constexpr (VB >= 4) {
      if (__builtin_expect(__builtin_fabsf(scale) < 0x1p100f, 1)) {
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
        return;
      }
    }
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
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float scale, float bias) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t q = (raw[e / 16] >> (2 * (e % 16))) & 0x3u;
      acc[e] = __builtin_fmaf(scale, (float)q, acc[e] + bias);
    }
  }
};

template <int VB>
struct Accum<ST_FP16, VB> {
  static constexpr int E = VB / 2;
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float x = (e & 1) ? half_hi(raw[e / 2]) : half_lo(raw[e / 2]);
      acc[e] = __builtin_fmaf(w, x, acc[e]);
    }
  }
};

template <int VB>
struct Accum<ST_BF16, VB> {
  static constexpr int E = VB / 2;
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint32_t u = (e & 1) ? (raw[e / 2] & 0xffff0000u) : (raw[e / 2] << 16);
      acc[e] = __builtin_fmaf(w, bits_to_float(u), acc[e]);
    }
  }
};

template <int VB>
struct Accum<ST_FP32, VB> {
  static constexpr int E = VB / 4;
  __device__ __forceinline__ static void run(float (&acc)[E], const uint32_t* raw, float w, float) {
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = __builtin_fmaf(w, bits_to_float(raw[e]), acc[e]);
  }
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
#pragma unroll
      for (int e = 0; e + 1 < E; e += 2) {
        const uint32_t lo = bf ? to_bf16_bits(acc[e]) : to_half_bits(acc[e]);
        const uint32_t hi = bf ? to_bf16_bits(acc[e + 1]) : to_half_bits(acc[e + 1]);
        w[e / 2] = lo | (hi << 16);
      }
      store_words<E * 2>(o, w);
    } else {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (col0 + e < D) o[e] = (uint16_t)(bf ? to_bf16_bits(acc[e]) : to_half_bits(acc[e]));
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

// One wave pools 64 / lanes bags of one table, `RN` entries of every bag per
// round.
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
template <typename index_t, int TY, int VB, int ROUND>
__device__ __forceinline__ void pool_bags(const LookupArgs& a, const TableDesc& d, int table, int first_slot,
                                          int lane, StageRow* stage_row, StageMul* stage_mul) {
  constexpr int BITS = type_bits(TY);
  constexpr int E = VB * 8 / BITS;
  constexpr int NW = (VB + 3) / 4;
  constexpr bool QUANT = TY == ST_INT8 || TY == ST_INT4 || TY == ST_INT2;
  constexpr bool ALIGNED = VB >= 4;
  constexpr int MAXR = 2; // entries one staging lane handles per round, at most

  const int S = d.lanes;
  const int G = 64 / S;
  const int grp = lane / S;
  const int sub = lane - grp * S;
  const int slot = first_slot + grp;
  const bool bag_ok = grp < G && slot < a.B;
  const bool reporter = sub == 0;
  // Entries staged per bag and round: ROUND, or half of it for bags that only
  // have two or three lanes (each staging lane handles at most MAXR entries).
  const int RN = S >= 4 ? ROUND : ROUND / 2;
  const int SL = S >= RN ? RN : (S >= 4 ? 4 : 2); // staging lanes per bag (power of two, <= S)
  const int R = RN / SL;                          // entries per staging lane per round
  const bool stager = bag_ok && sub < SL;

  // Bags are taken in the order the scheduler left them (longest first), so
  // that the bags sharing a wave have nearly equal lengths.
  int bag = slot;
  if (bag_ok && a.order) bag = a.order[(int64_t)table * a.B + slot];

  // Positions are counted the way the reference counts `current`: relative to
  // the first offset of the table's slice.
  int64_t pos0 = 0;
  int64_t len = 0;
  if (bag_ok) {
    const int64_t ob = (int64_t)table * a.B;
    const int64_t base = read_offset(a.offsets, a.off64, ob);
    const int64_t o0 = read_offset(a.offsets, a.off64, ob + bag);
    const int64_t o1 = read_offset(a.offsets, a.off64, ob + bag + 1);
    pos0 = a.check_total ? o0 - base : o0; // table-batched calls index the shared array
    len = o1 - o0;
    if (len < 0) {
      if (reporter) report(a.status, ERR_NEGATIVE_LENGTH);
      len = 0;
    }
    if (len > 0x7fffffffLL || pos0 < 0 || pos0 + len > a.index_size) {
      if (reporter) report(a.status, ERR_BAG_OVERRUN);
      len = 0;
    }
    if (a.check_total && bag == a.B - 1 && o1 - base != a.index_size && reporter)
      report(a.status, ERR_LENGTH_MISMATCH);
  }
  const int n = (int)len; // same for every lane of the bag

  const index_t* idx = reinterpret_cast<const index_t*>(a.indices);
  const uint8_t* wbase = (d.placement ? a.weights[1] : a.weights[0]) + d.weights_offset;
  const uint8_t* psb = wbase + d.sb_off;
  StageRow* my_row = stage_row + grp * RN;
  StageMul* my_mul = stage_mul + grp * RN;
  // the reference keeps the bag length in an int when it forms 1/len
  const float inv_len = (a.normalize && n > 0) ? 1.0f / (float)n : 1.0f;

  for (int pass = 0; pass < d.passes; ++pass) {
    const int chunk = pass * S + sub;
    const int byte_off = chunk * VB;
    const bool lane_on = bag_ok && byte_off < d.data_bytes;
    const uint8_t* pdata = wbase + d.data_off + byte_off;

    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.0f;

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
          if (a.sample_weights) nw[rr] = a.sample_weights[a.positional ? (int64_t)i : pos0 + i];
        }
      }
    };
    // index -> row offset, or "nothing to add"; publish the offsets of `round`
    auto stage_rows = [&](int round) {
#pragma unroll
      for (int rr = 0; rr < MAXR; ++rr) {
        int64_t row = nrow[rr];
        int64_t off = -1;
        if (rr < R && row != NO_ENTRY) {
          const int64_t pos = pos0 + round * RN + sub + rr * SL;
          bool ok = true;
          if (a.remap) {
            if (row < 0 || row >= a.remap_rows) {
              if (pass == 0) report_index(a.status, pos);
              ok = false;
            } else {
              row = (int64_t)a.remap[row];
              ok = row != -1;
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
          my_row[sub + rr * SL].off = off;
          if constexpr (!QUANT) {
            StageMul m;
            m.scale = nw[rr];
            m.bias = 0.0f;
            my_mul[sub + rr * SL] = m;
          }
        }
      }
    };

    load_idx(0);
    stage_rows(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    for (int r = 0; r * RN < n; ++r) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      uint32_t raw[ROUND][NW];
      uint32_t h0[MAXR], h1[MAXR];
      uint32_t valid = 0;
      const int left = min(n - r * RN, RN);
      // scale/bias first, so that their wait does not cover the row loads
      if constexpr (QUANT) {
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
#pragma unroll
      for (int e = 0; e < ROUND; ++e) {
        if (e < left) {
          const int64_t off = my_row[e].off;
          if (lane_on && off >= 0) {
            valid |= 1u << e;
            load_raw<VB>(raw[e], pdata + off);
          }
        }
      }
      load_idx(r + 1);
      if constexpr (QUANT) {
#pragma unroll
        for (int rr = 0; rr < MAXR; ++rr) {
          if (rr < R && stager && coff[rr] >= 0) {
            const float rs = d.sb_fp32 ? bits_to_float(h0[rr]) : half_lo(h0[rr]);
            const float rb = d.sb_fp32 ? bits_to_float(h1[rr]) : half_hi(h0[rr]);
            StageMul m;
            m.scale = cw[rr] * rs;
            m.bias = cw[rr] * rb;
            my_mul[sub + rr * SL] = m;
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      float sc[ROUND], bi[ROUND];
#pragma unroll
      for (int e = 0; e < ROUND; ++e) {
        if (e < left) {
          const StageMul m = my_mul[e];
          sc[e] = m.scale;
          bi[e] = m.bias;
        }
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int e = 0; e < ROUND; ++e) {
        if (valid & (1u << e)) Accum<TY, VB>::run(acc, raw[e], sc[e], bi[e]);
      }
      // offsets (and plain weights) of the next round; the column lanes have
      // read this round's entries by now
      stage_rows(r + 1);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }

    if (lane_on) {
      if (a.normalize && n > 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] *= inv_len;
      }
      const int col0 = chunk * E;
      const int64_t elem_pos = (int64_t)bag * a.out_stride + d.out_col + col0;
      const bool vec_ok = a.out_aligned && ((d.vec_store >> (a.out_ty == ST_FP32 ? 0 : 1)) & 1);
      write_out<E>(a, acc, elem_pos, col0, d.D, vec_ok);
    }
  }
}

template <typename index_t, int TY>
__device__ __forceinline__ void pool_dispatch_vb(const LookupArgs& a, const TableDesc& d, int table, int first_slot,
                                                 int lane, StageRow* stage_row, StageMul* stage_mul) {
  constexpr int BITS = type_bits(TY);
  constexpr int MINVB = BITS >= 16 ? BITS / 8 : 1;
#ifdef FBGEMM_AMD_ONLY_VB
  if (d.vb == FBGEMM_AMD_ONLY_VB) pool_bags<index_t, TY, FBGEMM_AMD_ONLY_VB, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
#else
  if (d.vb == 16) {
    if constexpr (TY == ST_INT2) pool_bags<index_t, TY, 4, 8>(a, d, table, first_slot, lane, stage_row, stage_mul); // not selected by the host
    else pool_bags<index_t, TY, 16, (TY == ST_INT4 ? 4 : 8)>(a, d, table, first_slot, lane, stage_row, stage_mul);
  } else if (d.vb == 4) {
    pool_bags<index_t, TY, 4, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
  } else {
    pool_bags<index_t, TY, MINVB, 8>(a, d, table, first_slot, lane, stage_row, stage_mul);
  }
#endif
}

template <typename index_t>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void lookup_kernel(const LookupArgs a) {
  __shared__ StageRow stage_rows_all[4][MAX_GROUPS * MAX_ROUND];
  __shared__ StageMul stage_muls_all[4][MAX_GROUPS * MAX_ROUND];
  const int lane = threadIdx.x & 63;
  const int wid = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  int64_t wave;
  if (a.xcd_start) {
    // Workgroups are handed to the 8 XCDs round-robin, so the workgroups with
    // id % 8 == x all run on one XCD and share its L2. Each XCD walks its own
    // run of the work list: whole tables (or slices of them) are pinned to
    // one L2 instead of spreading their hot rows over all eight.
    const int x = blockIdx.x & 7;
    const int64_t w = (int64_t)(blockIdx.x >> 3) * 4 + wid;
    const int64_t lo = a.xcd_start[x], hi = a.xcd_start[x + 1];
    if (w >= hi - lo) return;
    wave = lo + w;
  } else {
    wave = (int64_t)blockIdx.x * 4 + wid;
    if (wave >= a.num_waves) return;
  }
  StageRow* stage_row = stage_rows_all[wid];
  StageMul* stage_mul = stage_muls_all[wid];
  int table = 0, first_slot;
  if (a.work) {
    const WaveWork ww = a.work[wave];
    table = ww.table;
    first_slot = ww.first_bag;
  } else {
    first_slot = (int)(wave * (64 / a.single.lanes));
  }
  const TableDesc d = a.tables ? a.tables[table] : a.single;
#ifdef FBGEMM_AMD_ONLY_TY // register-budget experiments: compile a single row type
  if (d.ty == FBGEMM_AMD_ONLY_TY) pool_dispatch_vb<index_t, FBGEMM_AMD_ONLY_TY>(a, d, table, first_slot, lane, stage_row, stage_mul);
#else
  switch (d.ty) {
    case ST_INT4: pool_dispatch_vb<index_t, ST_INT4>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_INT8: pool_dispatch_vb<index_t, ST_INT8>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_FP16: pool_dispatch_vb<index_t, ST_FP16>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_INT2: pool_dispatch_vb<index_t, ST_INT2>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_FP32: pool_dispatch_vb<index_t, ST_FP32>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    case ST_BF16: pool_dispatch_vb<index_t, ST_BF16>(a, d, table, first_slot, lane, stage_row, stage_mul); break;
    default: break;
  }
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

__global__ __launch_bounds__(1024) void bag_order_kernel(const void* offsets, int off64, int32_t B, int32_t* order) {
  __shared__ int bins[SORT_BINS];
  __shared__ int partial[1024];
  const int t = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t ob = (int64_t)t * B;
  for (int i = tid; i < SORT_BINS; i += 1024) bins[i] = 0;
  __syncthreads();
  auto bin_of = [&](int b) {
    int64_t len = read_offset(offsets, off64, ob + b + 1) - read_offset(offsets, off64, ob + b);
    if (len < 0) len = 0;
    if (len > SORT_BINS - 1) len = SORT_BINS - 1;
    return SORT_BINS - 1 - (int)len; // longest first
  };
  for (int b = tid; b < B; b += 1024) atomicAdd(&bins[bin_of(b)], 1);
  __syncthreads();
  // exclusive scan of the SORT_BINS (== blockDim) counters
  const int mine = bins[tid];
  partial[tid] = mine;
  __syncthreads();
  for (int step = 1; step < 1024; step <<= 1) {
    const int v = tid >= step ? partial[tid - step] : 0;
    __syncthreads();
    partial[tid] += v;
    __syncthreads();
  }
  bins[tid] = partial[tid] - mine;
  __syncthreads();
  for (int b = tid; b < B; b += 1024) {
    const int p = atomicAdd(&bins[bin_of(b)], 1);
    order[ob + p] = b;
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
    if (mapped) v = (index_t)remap[rs + v];
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
  const int64_t blocks = a.xcd_start ? 8 * ((a.num_waves + 3) / 4) : (a.num_waves + 3) / 4;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  if (idx64) hipLaunchKernelGGL(lookup_kernel<int64_t>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(lookup_kernel<int32_t>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_bag_order(const void* offsets, bool off64, int32_t B, int32_t T, int32_t* order, hipStream_t stream) {
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
