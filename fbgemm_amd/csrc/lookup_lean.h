// The lean pooled-lookup kernel: the shapes that carry the traffic.
//
// Rows of 4-bit, 8-bit or fp16 elements whose data is a whole number of
// 16-byte chunks at 4-byte alignment, every lane owning 32 output columns of
// its bag (1, 2 or 4 chunks). Everything else (odd widths, unaligned tables,
// column passes, positional weights, 2-bit / fp32 / bf16 / fp8 rows) stays with
// the general kernel of lookup_general.h; the host decides per table
// (lean_shape in c_api.cpp).
//
// Same lane mapping and the same two row layouts as the general kernel: `lanes`
// consecutive lanes share a bag; either every lane loads data chunks and a
// staging lane fetches the row's (scale, bias) pair, or (inline_hdr) the lanes
// own 16-byte chunks of the whole row and the header rides in chunk 0. What is
// different:
//  * entries are staged 8 per bag at a time whatever the round size, so a line
//    of indices or per-sample weights is asked for at most twice instead of
//    once per round of 2 or 4 rows;
//  * the rows of a bag arrive through a software pipeline (pool_lean): units of
//    2 or 4 sixteen-byte loads per lane in two register sets that take turns,
//    the next block's row numbers staged in a second LDS buffer while the
//    current block is added up; an entry that adds nothing loads a row the wave
//    fetches anyway and carries the multiplier (-0, -0, -0), so no load needs a
//    predicate. Blocks whose units all exist run a copy of the loop without
//    conditions round the loads;
//  * EXACT selects the arithmetic: true is the reference's sequence of
//    roundings, acc = fma(scale, q, acc + bias) per element
//    (src/RefImplementations.cc:1326-1333,1519-1527), bit-identical to the CPU
//    path; false adds the biases of a bag apart, acc = fma(scale, q, acc) and
//    one bsum += bias per row and lane, out = acc + bsum: a third fewer vector
//    instructions per 4-bit element, results within a few fp32 roundings of the
//    reference's (tolerance grade, selected per plan).
//  * a wave that meets a scale too large for the pre-scaled arithmetic (scale *
//    2^24 times a half-precision denormal) starts over in pool_lean_slow, a plain
//    row-at-a-time loop that converts integers to float before the fma. Both
//    round identically; the slow one only has to be correct.
//  * what is staged per entry is the row number (32 bits), not its byte offset.
// Three kinds of kernel are made from this file: lookup_lean_kernel (every shape,
// float output), its Q8 instances (the 8-bit pooled output quantized in the
// output stage, lean_store_q8) and lookup_lean_wide4_kernel with its redo kernel
// (one shape, four waves per SIMD).
#pragma once
#include "lookup_device.h"

namespace fbgemm_amd {

constexpr int LEAN_BLOCK = 8;   // entries of every bag staged at a time
constexpr int LEAN_LDS_WORDS = 2048; // LDS of a wave: 64 lanes * 32 columns of fp32 output

struct __attribute__((aligned(16))) LeanMul {
  float s24;  // w * scale * 2^24 (4- and 8-bit rows, pre-scaled route); w * scale (plain route); w (fp16 rows)
  float s20;  // w * scale * 2^20 (4-bit rows, pre-scaled route)
  float bias; // w * bias
  uint32_t hole; // 1: nothing to add (the entry is absent, pruned or rejected): s24 = s20 = bias = -0
};

// ---- per-chunk arithmetic -------------------------------------------------------
//
// 16 bytes of a row in raw[4]. PLAIN = false: the pre-scaled route, masks leave
// small integers in the halves of a register as half-precision denormals
// (q * 2^-24, or q * 2^-20 for the odd nibbles), which the fma widens exactly;
// m.s24 / m.s20 carry the matching powers of two. PLAIN = true: the same masks,
// then one exact multiply turns the denormal into the integer as a float and
// the fma takes the unscaled m.s24 (= w * scale): for scales whose product with
// 2^24 would overflow. Both round like fma(scale, float(q), ...).

template <bool EXACT, bool PLAIN>
__device__ __forceinline__ float lean_fma(float s, float qd, float acc, float bias, float up) {
  const float q = PLAIN ? qd * up : qd; // exact: a small integer times a power of two
  return EXACT ? __builtin_fmaf(s, q, acc + bias) : __builtin_fmaf(s, q, acc);
}

template <int TY, bool EXACT, bool PLAIN, int NACC>
__device__ __forceinline__ void lean_chunk(float (&acc)[NACC], int base, const uint32_t (&raw)[4], const LeanMul& m) {
  if constexpr (TY == ST_INT4) {
    const float sa = m.s24, sb = PLAIN ? m.s24 : m.s20;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t x = raw[w];
      const uint32_t y = x >> 8;
      const uint32_t a0 = x & 0x000f000fu; // nibbles 0, 4
      const uint32_t a1 = x & 0x00f000f0u; // nibbles 1, 5 (times 16)
      const uint32_t a2 = y & 0x000f000fu; // nibbles 2, 6
      const uint32_t a3 = y & 0x00f000f0u; // nibbles 3, 7 (times 16)
      float* c = acc + base + 8 * w;
      c[0] = lean_fma<EXACT, PLAIN>(sa, half_lo(a0), c[0], m.bias, 0x1p24f);
      c[1] = lean_fma<EXACT, PLAIN>(sb, half_lo(a1), c[1], m.bias, 0x1p20f);
      c[2] = lean_fma<EXACT, PLAIN>(sa, half_lo(a2), c[2], m.bias, 0x1p24f);
      c[3] = lean_fma<EXACT, PLAIN>(sb, half_lo(a3), c[3], m.bias, 0x1p20f);
      c[4] = lean_fma<EXACT, PLAIN>(sa, half_hi(a0), c[4], m.bias, 0x1p24f);
      c[5] = lean_fma<EXACT, PLAIN>(sb, half_hi(a1), c[5], m.bias, 0x1p20f);
      c[6] = lean_fma<EXACT, PLAIN>(sa, half_hi(a2), c[6], m.bias, 0x1p24f);
      c[7] = lean_fma<EXACT, PLAIN>(sb, half_hi(a3), c[7], m.bias, 0x1p20f);
    }
  } else if constexpr (TY == ST_INT8) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t lo = __builtin_amdgcn_perm(0u, raw[w], 0x0c010c00u); // bytes 0, 1
      const uint32_t hi = __builtin_amdgcn_perm(0u, raw[w], 0x0c030c02u); // bytes 2, 3
      float* c = acc + base + 4 * w;
      c[0] = lean_fma<EXACT, PLAIN>(m.s24, half_lo(lo), c[0], m.bias, 0x1p24f);
      c[1] = lean_fma<EXACT, PLAIN>(m.s24, half_hi(lo), c[1], m.bias, 0x1p24f);
      c[2] = lean_fma<EXACT, PLAIN>(m.s24, half_lo(hi), c[2], m.bias, 0x1p24f);
      c[3] = lean_fma<EXACT, PLAIN>(m.s24, half_hi(hi), c[3], m.bias, 0x1p24f);
    }
  } else { // fp16: acc = fma(w, x, acc), the reference's own sequence in either mode
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float* c = acc + base + 2 * w;
      c[0] = __builtin_fmaf(m.s24, half_lo(raw[w]), c[0]);
      c[1] = __builtin_fmaf(m.s24, half_hi(raw[w]), c[1]);
    }
  }
}

// What a lane knows about its bag before the first row.
struct LeanLane {
  int grp, sub;   // bag slot inside the wave, chunk position inside the bag's lanes
  int lgrp;       // the bag slot whose staging area the lane reads (lanes left over shadow the last one)
  bool bag_ok;    // the lane pools a bag
  bool idle;      // the lane is left over (no bag slot of its own)
  int bag;        // the bag's number inside its table
  int n;          // entries of the bag
  int64_t pos0;   // position of its first entry in the index array
  int64_t remap_base, remap_cap; // pruned table: its slice of the remap array
  int64_t rank_base;             // >= 0: the table's first rank record (its mapping is order-preserving)
  bool remapped;
};

template <typename index_t>
__device__ __forceinline__ LeanLane lean_lane(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane) {
  LeanLane L;
  const int S = d.lanes;
  const int G = d.bags;
  bool idle;
  const uint32_t recip = (uint32_t)d.lanes_recip; // divisions by S, exact for arguments up to 64
  if (S <= 16 && !d.packed) {
    // quarter q of the wave holds bags q * (16 / S) ...; its last 16 % S lanes are left over
    const int per_q = G >> 2;
    const int j = lane & 15;
    const int gq = (int)(((uint32_t)j * recip) >> 16);
    idle = gq >= per_q;
    L.grp = (lane >> 4) * per_q + (idle ? per_q - 1 : gq);
    L.sub = j - gq * S;
  } else {
    L.grp = (int)(((uint32_t)lane * recip) >> 16);
    L.sub = lane - L.grp * S;
    idle = L.grp >= G;
  }
  const int slot = first_slot + L.grp;
  L.lgrp = idle ? G - 1 : L.grp;
  L.idle = idle;
  L.bag_ok = !idle && slot < a.B;
  const bool reporter = L.sub == 0;
  L.bag = slot;
  L.pos0 = 0;
  int64_t len = 0;
  if (L.bag_ok) {
    const int64_t ob = (int64_t)table * a.B;
    int64_t o0, o1;
    if (a.order) {
      const BagEntry be = a.order[ob + slot];
      L.bag = be.bag;
      o0 = be.o0;
      o1 = o0 + be.len;
      if (be.len < 0) { // a length the entry cannot hold: judge the offsets themselves
        o0 = read_offset(a.offsets, a.off64, ob + be.bag);
        o1 = read_offset(a.offsets, a.off64, ob + be.bag + 1);
      }
    } else {
      o0 = read_offset(a.offsets, a.off64, ob + slot);
      o1 = read_offset(a.offsets, a.off64, ob + slot + 1);
    }
    int64_t base = 0;
    if (a.check_total) base = read_offset(a.offsets, a.off64, ob);
    L.pos0 = o0 - base; // table-batched calls index the shared array: base = 0
    len = o1 - o0;
    if (len < 0) {
      if (reporter) report(a.status, ERR_NEGATIVE_LENGTH);
      len = 0;
    }
    if (len > 0x7fffffffLL || L.pos0 < 0 || L.pos0 + len > a.index_size) {
      if (reporter) report(a.status, ERR_BAG_OVERRUN);
      len = 0;
    }
    if (a.check_total && L.bag == a.B - 1 && o1 - base != a.index_size && reporter) report(a.status, ERR_LENGTH_MISMATCH);
  }
  L.n = (int)len;
  L.remap_base = 0;
  L.remap_cap = 0;
  L.rank_base = -1;
  L.remapped = false;
  if (a.remap) {
    L.remapped = true;
    L.remap_cap = a.remap_rows;
    if (a.remap_offsets) {
      L.remap_base = a.remap_offsets[table];
      L.remap_cap = a.remap_offsets[table + 1] - L.remap_base;
      L.remapped = L.remap_cap > 0;
      if (a.rank_records) L.rank_base = a.rank_offsets[table];
    }
  }
  return L;
}

// Largest of a non-negative value over the wave, through lane shifts inside the
// rows of 16 and the two row broadcasts (six vector instructions, no LDS).
__device__ __forceinline__ int lean_wave_max(int v) {
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false)); // row_shr:1
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false)); // row_shr:2
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false)); // row_shr:4
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false)); // row_shr:8: lane 15 of a row holds the row's largest
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false)); // row_bcast:15 into rows 1 and 3
  v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false)); // row_bcast:31 into rows 2 and 3
  return __builtin_amdgcn_readlane(v, 63);
}

constexpr int LEAN_NO_ENTRY = INT32_MIN;  // the bag has no such entry
constexpr int LEAN_SKIP = -1;             // an entry that adds nothing (a pruned or rejected row)

// index -> row number, LEAN_SKIP for what the reference skips or rejects. A rejected index
// leaves its position in `bad_pos` (the smallest wins); the caller reports it once its loop is
// over (lean_report_bad): an atomic inside the loop would count as a store in flight, and with
// loads and stores in flight together every wait of the loop becomes a wait for everything.
constexpr int64_t LEAN_NO_BAD_POS = INT64_MAX;
__device__ __forceinline__ int lean_row(const TableDesc& d, const LeanLane& L, int64_t row, int64_t pos, int64_t& bad_pos) {
  if (!L.remapped && d.skip_minus_one && row == -1) return LEAN_SKIP;
  if (row < 0 || row >= d.num_rows) {
    bad_pos = pos < bad_pos ? pos : bad_pos;
    return LEAN_SKIP;
  }
  return (int)row;
}
constexpr int64_t LEAN_PRUNED = INT64_MIN; // what lean_remap returns for an entry that adds nothing
__device__ __forceinline__ int64_t lean_remap(const LookupArgs& a, const LeanLane& L, int64_t logical, int64_t pos, int64_t& bad_pos) {
  if (logical < 0 || logical >= L.remap_cap) {
    bad_pos = pos < bad_pos ? pos : bad_pos;
    return LEAN_PRUNED;
  }
  if (L.rank_base >= 0) { // order-preserving mapping: the physical row is the rank among the kept rows
    const RankRecord r = a.rank_records[L.rank_base + (logical >> 5)];
    const uint32_t bit = (uint32_t)logical & 31u;
    if (!((r.bits >> bit) & 1u)) return LEAN_PRUNED;
    return (int64_t)(r.before + (uint32_t)__builtin_popcount(r.bits & ((1u << bit) - 1u)));
  }
  const int64_t m = a.remap64 ? reinterpret_cast<const int64_t*>(a.remap)[L.remap_base + logical]
                              : (int64_t) reinterpret_cast<const int32_t*>(a.remap)[L.remap_base + logical];
  return m == -1 ? LEAN_PRUNED : m;
}
__device__ __forceinline__ void lean_report_bad(const LookupArgs& a, int64_t bad_pos) {
  if (bad_pos != LEAN_NO_BAD_POS) report_index(a.status, bad_pos);
}

// The output of a wave through LDS, so that every store instruction writes runs
// of consecutive bytes: a lane holds 32 consecutive columns of its bag (64 or 128
// bytes of output), and storing them lane by lane would put the lanes of one
// instruction 64 or 128 bytes apart, four or eight partial writes to every line.
// Here the lanes of a bag first leave their 16-byte pieces in LDS in column order
// and then take them back interleaved: piece sub, sub + lanes, sub + 2 lanes, ...,
// which makes each instruction write lanes * 16 consecutive bytes per bag.
// ESZ: bytes per output element. `lds` must hold the wave's whole output (at most
// 64 lanes * 32 columns * 4 bytes = LEAN_LDS_WORDS) and MAX_GROUPS words behind it, and is
// free once the last block is pooled.
template <int TY, int C, bool INHDR, int ESZ>
__device__ __forceinline__ void lean_store_interleaved(const LookupArgs& a, const TableDesc& d, const LeanLane& L,
                                                       const float (&acc)[C * (TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8))],
                                                       uint32_t* lds) {
  constexpr int E = TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8);
  // whole-row chunks start E / 4 columns before a multiple of E: pieces of 8 bytes where that is not 16 bytes
  constexpr int PB = (INHDR && (E / 4 * ESZ) % 16 != 0) ? 8 : 16;
  constexpr int WP = PB / 4;           // words per piece
  constexpr int NP = E * ESZ / PB;     // pieces per chunk
  constexpr int SHIFT = INHDR ? (E / 4 * ESZ) / PB : 0;
  const int S = d.lanes;
  const int npb = d.D * ESZ / PB;      // pieces of a bag's block of the output
  uint32_t* mine = lds + (size_t)L.grp * npb * WP;
  const bool bf = a.out_ty == ST_BF16;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    uint32_t w[E * ESZ / 4];
    if constexpr (ESZ == 4) {
#pragma unroll
      for (int e = 0; e < E; ++e) w[e] = float_to_bits(acc[c * E + e]);
    } else {
      if (bf) {
#pragma unroll
        for (int e = 0; e < E; e += 2) w[e / 2] = pack_bf16x2(acc[c * E + e], acc[c * E + e + 1]);
      } else {
#pragma unroll
        for (int e = 0; e < E; e += 2) w[e / 2] = pack_half2(acc[c * E + e], acc[c * E + e + 1]);
      }
    }
    const int g0 = (L.sub + c * S) * NP - SHIFT;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int gq = g0 + q;
      if (L.bag_ok && gq >= 0 && gq < npb) {
        if constexpr (WP == 4) *reinterpret_cast<uint4*>(mine + gq * 4) = make_uint4(w[4 * q], w[4 * q + 1], w[4 * q + 2], w[4 * q + 3]);
        else *reinterpret_cast<uint2*>(mine + gq * 2) = make_uint2(w[2 * q], w[2 * q + 1]);
      }
    }
  }
  // the bag every group of the wave writes for (-1: none), behind the pieces
  int* bag_of = reinterpret_cast<int*>(lds + LEAN_LDS_WORDS);
  if (L.sub == 0 && !L.idle) bag_of[L.grp] = L.bag_ok ? L.bag : -1;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int64_t row_bytes = a.out_stride * ESZ;
  uint8_t* out0 = reinterpret_cast<uint8_t*>(a.out) + (int64_t)d.out_col * ESZ;
  if ((npb & (npb - 1)) == 0 && S < 8) {
    // The pieces of the whole wave, bag after bag, dealt to the lanes in that order: consecutive
    // lanes write consecutive pieces of one bag, so a store instruction covers whole runs of a
    // bag's block (all of it when the block has no more than 64 pieces) instead of `lanes` pieces
    // of every bag, which for bags of 2..4 lanes are fragments of 32..64 bytes that reach memory
    // as partial writes of their lines. (Bags of 8 lanes and more write runs of 128 bytes either
    // way and keep the mapping below, which needs no look-up of the bag: 2.5 % on the HBM-sized
    // configuration.)
    const int shift = __builtin_ctz((unsigned)npb);
    const int total = d.bags << shift;
#pragma unroll
    for (int it = 0; it < C * NP; ++it) {
      const int f = (int)threadIdx.x + it * 64;
      if (f < total) {
        const int g = f >> shift;
        const int piece = f & (npb - 1);
        const int bag = bag_of[g];
        if (bag >= 0) {
          uint8_t* dst = out0 + (int64_t)bag * row_bytes + (size_t)piece * PB;
          // streaming stores: whole runs of the output, written once and never read back here
          if constexpr (WP == 4) {
            const uint4 v = *reinterpret_cast<const uint4*>(lds + (size_t)f * 4);
            stream_store16(dst, v.x, v.y, v.z, v.w);
          } else {
            const uint2 v = *reinterpret_cast<const uint2*>(lds + (size_t)f * 2);
            stream_store8(dst, v.x, v.y);
          }
        }
      }
    }
    return;
  }
  uint8_t* block = out0 + (int64_t)L.bag * row_bytes;
#pragma unroll
  for (int it = 0; it < C * NP; ++it) {
    const int gq = L.sub + it * S;
    if (L.bag_ok && gq < npb) {
      if constexpr (WP == 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(mine + gq * 4);
        stream_store16(block + (size_t)gq * 16, v.x, v.y, v.z, v.w);
      } else {
        const uint2 v = *reinterpret_cast<const uint2*>(mine + gq * 2);
        stream_store8(block + (size_t)gq * 8, v.x, v.y);
      }
    }
  }
}

// The 8-bit pooled output (output type ST_INT8 of a table-batched forward): the bag's block of
// the line is the pooled fp32 vector quantized row-wise to 8 bits, D bytes followed by an fp32
// scale and an fp32 bias, the block of table t starting 8 t bytes behind its float column (the
// reference operator's output stage, embedding_forward_quantized_split_nbit_kernel_template.cu:
// 535-560; the arithmetic is the core library's FloatToFused8BitRowwiseQuantizedSBFloat,
// src/QuantUtils.cc:677-718, which is what the reference's test expects of it and what
// quantize_rowwise_kernel computes from a float forward):
//   scale = (max - min) / 255, bias = min, q = lrintf((x - min) * (255 / (max - min + 1e-8))),
// min and max being the FIRST smallest / largest element of the block, which only shows when
// the extreme is a zero and zeros of both signs are in the block.
// `pooled` holds the wave's pooled vectors, D floats per bag slot (lean_store_q8 puts them
// there). The lanes of a bag take groups of 4 columns in turn, so one store instruction writes
// 4 * lanes consecutive bytes per bag, and exchange their extremes by lane shuffles (any number
// of lanes per bag). One copy of this code serves every row type.
__device__ __forceinline__ void lean_q8_from_lds(const LookupArgs& a, const TableDesc& d, const LeanLane& L, int table,
                                                 const float* pooled) {
  const int S = d.lanes, D = d.D;
  const int base = (int)threadIdx.x - L.sub; // first lane of the bag
  const float* mine = pooled + (size_t)L.grp * D;
  // whole groups of 4 columns, read as 16 bytes (every bag's floats start at a multiple of 16 bytes
  // when D is a multiple of 4; otherwise all columns are lane 0's, one by one)
  const int nq = (D & 3) == 0 ? D >> 2 : 0;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  auto see = [&](float x) {
    lo = x < lo ? x : lo;
    hi = hi < x ? x : hi;
  };
  for (int q = L.sub; q < nq; q += S) {
    const float4 v = *reinterpret_cast<const float4*>(mine + 4 * q);
    see(v.x);
    see(v.y);
    see(v.z);
    see(v.w);
  }
  if (L.sub == 0)
    for (int c = nq * 4; c < D; ++c) see(mine[c]);
  for (int j = 0; j < S; ++j) {
    const float ol = __shfl(lo, base + j, 64), oh = __shfl(hi, base + j, 64);
    lo = ol < lo ? ol : lo;
    hi = hi < oh ? oh : hi;
  }
  float minimum = lo, maximum = hi;
  if (__builtin_amdgcn_ballot_w64(L.bag_ok && (lo == 0.0f || hi == 0.0f)) != 0ull) {
    // A zero extreme: every element is on one side of it, so the first of the equal extremes is
    // the first zero of the block, of either sign (positions compared), and it is the same
    // element for the minimum and for the maximum when both are zero.
    constexpr int NONE = 0x7fffffff;
    int zi = NONE;
    float zv = 0.0f;
    auto zero_at = [&](float x, int col) {
      if (zi == NONE && x == 0.0f) {
        zi = col;
        zv = x;
      }
    };
    for (int q = L.sub; q < nq; q += S) {
      const float4 v = *reinterpret_cast<const float4*>(mine + 4 * q);
      zero_at(v.x, 4 * q);
      zero_at(v.y, 4 * q + 1);
      zero_at(v.z, 4 * q + 2);
      zero_at(v.w, 4 * q + 3);
    }
    if (L.sub == 0)
      for (int c = nq * 4; c < D; ++c) zero_at(mine[c], c);
    const int my_zi = zi;
    const float my_zv = zv;
    for (int j = 0; j < S; ++j) {
      const int oi = __shfl(my_zi, base + j, 64);
      const float ov = __shfl(my_zv, base + j, 64);
      if (oi < zi) {
        zi = oi;
        zv = ov;
      }
    }
    if (lo == 0.0f && zi != NONE) minimum = zv;
    if (hi == 0.0f && zi != NONE) maximum = zv;
  }
  if (!L.bag_ok) return;
  const float range = maximum - minimum;
  const float inverse_scale = 255.0f / (range + 1e-8f);
  auto quant = [&](float x) { return (uint32_t)(int)__builtin_rintf((x - minimum) * inverse_scale) & 0xffu; }; // to nearest, ties to even
  uint8_t* row = reinterpret_cast<uint8_t*>(a.out) + (int64_t)L.bag * a.out_stride + d.out_col + 8 * (int64_t)table;
  const bool words = (reinterpret_cast<uintptr_t>(row) & 3) == 0;
  for (int q = L.sub; q < nq; q += S) {
    const float4 v = *reinterpret_cast<const float4*>(mine + 4 * q);
    const uint32_t w = quant(v.x) | (quant(v.y) << 8) | (quant(v.z) << 16) | (quant(v.w) << 24);
    if (words) {
      *reinterpret_cast<uint32_t*>(row + 4 * q) = w;
    } else {
      for (int k = 0; k < 4; ++k) row[4 * q + k] = (uint8_t)(w >> (8 * k));
    }
  }
  if (L.sub == 0) {
    for (int c = nq * 4; c < D; ++c) row[c] = (uint8_t)quant(mine[c]);
    const uint32_t sb[2] = {float_to_bits(range / 255.0f), float_to_bits(minimum)};
    uint8_t* p = row + D;
    if ((reinterpret_cast<uintptr_t>(p) & 3) == 0) {
      reinterpret_cast<uint32_t*>(p)[0] = sb[0];
      reinterpret_cast<uint32_t*>(p)[1] = sb[1];
    } else {
      for (int b = 0; b < 8; ++b) p[b] = (uint8_t)(sb[b >> 2] >> (8 * (b & 3)));
    }
  }
}

// The pooled vectors of the wave into LDS, D floats per bag slot, then lean_q8_from_lds. `lds`
// must hold the wave's whole output as floats (at most 64 lanes * 32 columns = LEAN_LDS_WORDS)
// and is free once the last block is pooled.
template <int TY, int C, bool INHDR>
__device__ __forceinline__ void lean_store_q8(const LookupArgs& a, const TableDesc& d, const LeanLane& L, int table,
                                              const float (&acc)[C * (TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8))], uint32_t* lds) {
  constexpr int E = TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8);
  const int S = d.lanes, D = d.D;
  float* mine = reinterpret_cast<float*>(lds) + (size_t)L.grp * D;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    // first column of the chunk (whole-row chunks start E / 4 columns early: the header)
    const int col0 = (L.sub + c * S) * E - (INHDR ? E / 4 : 0);
#pragma unroll
    for (int e = 0; e < E; e += 4) {
      const int col = col0 + e;
      if (!L.bag_ok || L.idle) continue;
      if (col >= 0 && col + 4 <= D && (D & 3) == 0) {
        *reinterpret_cast<float4*>(mine + col) = make_float4(acc[c * E + e], acc[c * E + e + 1], acc[c * E + e + 2], acc[c * E + e + 3]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (col + k >= 0 && col + k < D) mine[col + k] = acc[c * E + e + k];
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  lean_q8_from_lds(a, d, L, table, reinterpret_cast<const float*>(lds));
}

// VIA_LDS: floating-point output goes through lean_store_interleaved where its shape allows.
// Q8: the kernel instance that writes the 8-bit pooled output (and nothing else).
template <bool EXACT, int TY, int C, bool INHDR, bool VIA_LDS, bool Q8>
__device__ __forceinline__ void lean_write(const LookupArgs& a, const TableDesc& d, const LeanLane& L, int table, float (&acc)[C * (TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8))], float bsum, uint32_t* lds) {
  constexpr bool QUANT = TY == ST_INT8 || TY == ST_INT4;
  constexpr int E = TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8);
  constexpr int NACC = C * E;
  const bool vec_ok = a.out_aligned && ((d.vec_store >> (a.out_ty == ST_FP32 ? 0 : 1)) & 1);
  if constexpr (!EXACT && QUANT) {
#pragma unroll
    for (int e = 0; e < NACC; ++e) acc[e] += bsum;
  }
  if (a.normalize && L.n > 0) {
    const float inv_len = 1.0f / (float)L.n; // the reference keeps the bag length in an int when it forms 1/len
#pragma unroll
    for (int e = 0; e < NACC; ++e) acc[e] *= inv_len;
  }
  if constexpr (Q8) {
    lean_store_q8<TY, C, INHDR>(a, d, L, table, acc, lds);
    return;
  }
  // whole 16-byte (8-byte) pieces at aligned places: through LDS, interleaved
  if (VIA_LDS && vec_ok) {
    if (a.out_ty == ST_FP32) {
      if ((d.D * 4) % 16 == 0) {
        lean_store_interleaved<TY, C, INHDR, 4>(a, d, L, acc, lds);
        return;
      }
    } else if ((d.D * 2) % 16 == 0) {
      lean_store_interleaved<TY, C, INHDR, 2>(a, d, L, acc, lds);
      return;
    }
  }
  const int nchunks = INHDR ? (d.data_bytes + 4 + 15) / 16 : d.lanes * C;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int k = L.sub + c * d.lanes;
    if (L.bag_ok && k < nchunks) {
      float part[E];
#pragma unroll
      for (int e = 0; e < E; ++e) part[e] = acc[c * E + e];
      if constexpr (INHDR) {
        write_out_runs<E>(a, part, (int64_t)L.bag * a.out_stride + d.out_col, k * E - E / 4, d.D, vec_ok);
      } else {
        const int col0 = k * E;
        write_out<E>(a, part, (int64_t)L.bag * a.out_stride + d.out_col + col0, col0, d.D, vec_ok);
      }
    }
  }
}

// One wave pools bags_per_wave(lanes, packed) bags of one table.
// C: 16-byte chunks per lane and row (32 columns per lane: 1 for 4-bit, 2 for
// 8-bit, 4 for fp16 rows). INHDR as in the general kernel. R: entries a staging
// lane handles per block (8 / the staging lanes of a bag: 1 for bags of 8 lanes
// and more, 2 for 4..7 lanes, 4 for 2..3 lanes).
//
// The rows of a bag are fetched in units of 4 loads of 16 bytes per lane (4, 2 or
// 1 rows) into two register sets that take turns: while one unit is added up the
// other is in flight, and as soon as a set is free the unit after the next is
// asked for, so a lane has 4 to 8 loads outstanding at all times instead of 8
// while it waits and none while it computes. Units cross block boundaries: the
// rows of block k + 1 are staged (in the second of two LDS buffers) before the
// arithmetic of block k starts, its indices having been fetched a block earlier.
// Loads return in the order they were issued, so everything a step waits for is
// issued before what should stay in flight behind it:
//   iteration k:  multipliers of block k    <- headers(k), issued in iteration k - 1
//                 rows, weights of block k+1 <- indices(k+1), issued in iteration k - 1
//                 issue indices(k+2); stage the rows of block k+1; issue headers(k+1)
//                 for every unit of block k: add it up, issue the unit two further on
// An entry that adds nothing (absent, pruned, rejected) is staged as a row the
// wave has seen to be valid with the multiplier (-0, -0, -0), which leaves every
// accumulator as it is: the loads need no predicate. (Until the wave has seen a
// valid row its units are not loaded at all.)
// Returns false (wave-uniform, nothing written) when a scale is too large for
// the pre-scaled arithmetic.
template <typename index_t, bool EXACT, int TY, int C, bool INHDR, int R, bool Q8, int UL_CAP = 4, bool HDR_EARLY = false>
__device__ __forceinline__ bool pool_lean(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane,
                                          uint32_t* lds) {
  constexpr bool QUANT = TY == ST_INT8 || TY == ST_INT4;
  constexpr int E = TY == ST_INT4 ? 32 : (TY == ST_INT8 ? 16 : 8); // columns per chunk
  // 16-byte loads per lane and unit. 4 for fp16 rows (one row). Quantised rows: 2 with the exact
  // arithmetic, which is bound by the vector units and gains nothing from more loads in flight
  // (HBM-sized configuration: 2.97 ms with 2, 3.10 ms with 4); 4 with the tolerance-grade
  // arithmetic (2.71 against 2.76 ms), except where the staging lanes hold 4 entries each and
  // fetch the row headers: their registers and 4-load units together do not fit the 168
  // registers that 3 waves per SIMD leave a lane.
  constexpr int UL_RULE = !QUANT ? 4 : (EXACT || (R == 4 && !INHDR)) ? 2 : 4;
  constexpr int UL = UL_RULE < UL_CAP ? UL_RULE : UL_CAP;
  constexpr int HALF = UL / C;                                     // rows per unit
  constexpr int U = LEAN_BLOCK / HALF;                             // units per block
  constexpr int SL = LEAN_BLOCK / R;                               // staging lanes per bag
  constexpr int ROWS_BUF = MAX_GROUPS * LEAN_BLOCK;                // one buffer of staged rows
  static_assert(!INHDR || QUANT, "whole-row chunks belong to rows with a header");

  int* stage_row = reinterpret_cast<int*>(lds);                               // [2][MAX_GROUPS][LEAN_BLOCK]
  LeanMul* stage_mul = reinterpret_cast<LeanMul*>(lds + 2 * ROWS_BUF);        // [MAX_GROUPS][LEAN_BLOCK]

  const LeanLane L = lean_lane<index_t>(a, d, table, first_slot, lane);
  const int S = d.lanes;
  const int sub = L.sub;
  const int n = L.n;
  // every bag slot of the wave stages, also one past the table's last bag (its entries are all absent)
  const bool stager = !L.idle && sub < SL;
  // the longest bag of the wave bounds the loop (wave-uniform)
  const int nmax = lean_wave_max(n);
  const int units = (int)(((uint32_t)nmax + HALF - 1) / HALF);

  const index_t* idx = reinterpret_cast<const index_t*>(a.indices) + L.pos0;
  const float* sw = a.sample_weights ? a.sample_weights + L.pos0 : nullptr;
  const uint8_t* wbase = (d.placement ? a.weights[1] : a.weights[0]) + d.weights_offset;
  const uint8_t* psb = wbase + d.sb_off;
  const uint32_t stride = (uint32_t)d.row_stride;
  int* my_rows = stage_row + L.lgrp * LEAN_BLOCK;
  LeanMul* my_mul = stage_mul + L.lgrp * LEAN_BLOCK;
  // this lane's chunks of row 0; whole-row chunks: a slot past the row's last chunk
  // shadows it (same bytes, nothing written)
  const uint8_t* pchunk[C];
  if constexpr (INHDR) {
    const int nchunks = (d.data_bytes + 4 + 15) / 16;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int k = sub + c * S;
      pchunk[c] = wbase + (k < nchunks ? k : nchunks - 1) * 16;
    }
  } else {
#pragma unroll
    for (int c = 0; c < C; ++c) pchunk[c] = wbase + d.data_off + (sub + c * S) * 16;
  }

  float acc[C * E];
#pragma unroll
  for (int e = 0; e < C * E; ++e) acc[e] = 0.0f;
  float bsum = -0.0f; // tolerance grade: the biases of the bag, added once at the end

  // the two register sets of rows in flight
  uint32_t raw_a[HALF][C][4], raw_b[HALF][C][4];
#pragma unroll
  for (int e = 0; e < HALF; ++e)
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
      for (int w = 0; w < 4; ++w) raw_a[e][c][w] = raw_b[e][c][w] = 0u;

  // registers of the staging lanes: the indices and weights on their way, the rows
  // and weights of the block staged last, its headers on their way
  int64_t nrow[R];
  float nw[R];
  bool have[R];
  int crow[R];
  float cw[R];
  uint32_t h0[R], h1[R];
  int64_t bad_pos = LEAN_NO_BAD_POS; // the first rejected index this lane has met
  int safe = -1;         // a row of the table that can be loaded (wave-uniform); -1: none seen yet
  uint32_t loadable = 0; // bit p: the rows staged in buffer p can be loaded (wave-uniform)
  uint32_t holey = 0;    // bit p: some entry staged in buffer p adds nothing (wave-uniform; fp16 rows only)

  auto issue_idx = [&](int blk) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      nrow[j] = 0;
      nw[j] = 1.0f;
      const int i = blk * LEAN_BLOCK + sub + j * SL;
      have[j] = stager && i < n;
      if (have[j]) {
        nrow[j] = (int64_t)idx[i];
        if (sw) nw[j] = sw[i];
      }
    }
  };
  // indices that have arrived -> row numbers (negative: nothing to add), weights
  auto take_idx = [&](int blk) {
    if (L.remapped) {
#pragma unroll
      for (int j = 0; j < R; ++j)
        if (have[j]) nrow[j] = lean_remap(a, L, nrow[j], L.pos0 + blk * LEAN_BLOCK + sub + j * SL, bad_pos);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
      crow[j] = LEAN_NO_ENTRY;
      // a copy made here and now: left to itself the compiler keeps the weight where it was
      // loaded, loads the next block's weight elsewhere and moves both at the end of the loop,
      // which waits for that load and for everything issued before it
      asm volatile("v_mov_b32 %0, %1" : "=v"(cw[j]) : "v"(nw[j]));
      if (have[j]) crow[j] = nrow[j] == LEAN_PRUNED ? LEAN_SKIP : lean_row(d, L, nrow[j], L.pos0 + blk * LEAN_BLOCK + sub + j * SL, bad_pos);
    }
  };
  // The (scale, bias) headers of the rows staged last, asked for right in front of the first unit
  // of their block: a header sits in the line its row's data starts in, and asked for close to the
  // data the two requests merge (asked for a block earlier, at staging time, the line was often
  // gone again when the data loads came: 14 % more requests to L2 on the HBM-sized configuration).
  // Two shapes keep asking at staging time: 8-bit rows read as two chunks per lane with two or
  // four entries per staging lane have no registers to spare where the units are asked for, and
  // in the bit-exact mode with one entry per staging lane (eight or more lanes per bag) the
  // multipliers are wanted so soon after the short two-row units that the later request cost
  // 2 % where the merged requests saved 1 %.
  constexpr bool HDRS_WITH_UNITS = !(TY == ST_INT8 && C == 2 && R >= 2) && !(EXACT && R == 1) && !HDR_EARLY;
  auto issue_hdrs = [&]() {
    if constexpr (QUANT && !INHDR) {
#pragma unroll
      for (int j = 0; j < R; ++j) {
        h0[j] = h1[j] = 0u;
        if (crow[j] >= 0) {
          const uint8_t* ph = psb + (uint64_t)(uint32_t)crow[j] * stride;
          if (TY == ST_INT8 && d.sb_fp32) { // two floats behind the data: 8-bit rows of the single-table layout only
            const Dwordx2 v = *reinterpret_cast<const Dwordx2*>(ph);
            h0[j] = v.v[0];
            h1[j] = v.v[1];
          } else {
            h0[j] = *reinterpret_cast<const uint32_t*>(ph);
          }
        }
      }
    }
  };
  // the rows of block blk into buffer blk & 1
  auto stage_rows = [&](int blk) {
    int cand = -1;
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (crow[j] >= 0) cand = crow[j];
    const uint64_t seen = __builtin_amdgcn_ballot_w64(cand >= 0);
    if (seen != 0ull) safe = __builtin_amdgcn_readlane(cand, (int)__builtin_ctzll(seen));
    const int p = blk & 1;
    loadable = safe >= 0 ? (loadable | (1u << p)) : (loadable & ~(1u << p));
    if constexpr (!QUANT) {
      bool hole = false;
#pragma unroll
      for (int j = 0; j < R; ++j) hole = hole || crow[j] < 0;
      holey = __builtin_amdgcn_ballot_w64(stager && hole) != 0ull ? (holey | (1u << p)) : (holey & ~(1u << p));
    }
    if (stager) {
#pragma unroll
      for (int j = 0; j < R; ++j) my_rows[p * ROWS_BUF + sub + j * SL] = crow[j] >= 0 ? crow[j] : safe;
    }
    if constexpr (!HDRS_WITH_UNITS) issue_hdrs();
  };
  // the multipliers of the block whose rows were staged last; true: a scale too large for the pre-scaled route
  auto stage_muls = [&]() {
    bool big = false;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      LeanMul m;
      m.s24 = -0.0f;
      m.s20 = -0.0f;
      m.bias = -0.0f;
      m.hole = 1u;
      if (crow[j] >= 0) {
        m.hole = 0u;
        if constexpr (QUANT && !INHDR) {
          const bool pair32 = TY == ST_INT8 && d.sb_fp32;
          const float rs = pair32 ? bits_to_float(h0[j]) : half_lo(h0[j]);
          const float rb = pair32 ? bits_to_float(h1[j]) : half_hi(h0[j]);
          const float sc = cw[j] * rs;
          big = big || !(__builtin_fabsf(sc) < 0x1p100f);
          m.s24 = sc * 0x1p24f;
          m.s20 = sc * 0x1p20f;
          m.bias = cw[j] * rb;
        } else {
          // fp16 rows and whole-row chunks: the multiplier is the weight. Whole-row chunks take fp16
          // headers: |scale| <= 65504, so only a huge weight can overflow the pre-scaling
          m.s24 = cw[j];
          if constexpr (INHDR) big = big || !(__builtin_fabsf(cw[j]) < 0x1p60f);
        }
      }
      if (stager) my_mul[sub + j * SL] = m;
    }
    return big;
  };
  auto lds_sync = [&]() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // unit g (counted from the bag's first row) into one of the register sets; `live`: the rows of
  // the unit that some bag of the wave has (wave-uniform; the rest is neither loaded nor added)
  auto issue_unit = [&](uint32_t (&raw)[HALF][C][4], int g, int live) {
    const int* rows = my_rows + ((g / U) & 1) * ROWS_BUF + (g % U) * HALF;
#pragma unroll
    for (int e = 0; e < HALF; ++e) {
      if (e >= live) break;
      const uint64_t off = (uint64_t)(uint32_t)rows[e] * stride;
#pragma unroll
      for (int c = 0; c < C; ++c) load_raw<16>(raw[e][c], pchunk[c] + off);
    }
  };
  // unit u of the block whose multipliers are staged: added to the accumulators.
  // `holes`: the block may hold entries that add nothing (fp16 rows only: see below)
  auto add_unit = [&](uint32_t (&raw)[HALF][C][4], int u, bool holes, int live) {
#pragma unroll
    for (int e = 0; e < HALF; ++e) {
      if (e >= live) break;
      LeanMul m = my_mul[u * HALF + e];
      if constexpr (INHDR) {
        // the row header sits in the first dword of chunk 0, which the first lane of the group
        // holds; an entry that adds nothing has loaded some other row: its header does not count
        uint32_t h = (uint32_t)__builtin_amdgcn_ds_bpermute((lane - sub) * 4, (int)raw[e][0][0]);
        h = m.hole ? 0u : h;
        const float sc = m.s24 * half_lo(h);
        m.bias = m.s24 * half_hi(h);
        m.s24 = sc * 0x1p24f;
        m.s20 = sc * 0x1p20f;
      }
      if constexpr (!QUANT) {
        // the row an absent entry has loaded may hold infinities: -0 times them is not nothing
        if (holes && m.hole) {
#pragma unroll
          for (int c = 0; c < C; ++c)
#pragma unroll
            for (int w = 0; w < 4; ++w) raw[e][c][w] = 0u;
        }
      }
      if constexpr (!EXACT && QUANT) bsum += m.bias;
#pragma unroll
      for (int c = 0; c < C; ++c) lean_chunk<TY, EXACT, false, C * E>(acc, c * E, raw[e][c], m);
    }
  };
  auto can_load = [&](int g) { return g < units && ((loadable >> ((g / U) & 1)) & 1u) != 0u; };
  // rows of unit g that the longest bag of the wave has: HALF but for the last unit. (Units of 4
  // rows only: 1.8 % on the HBM-sized configuration in the tolerance-grade mode, where a bag of 15
  // rows otherwise pays for 16. With units of 2 rows the test per row costs more than the row
  // saved now and then: the exact mode lost 3.8 % to it.)
  auto live_rows = [&](int g) { return (HALF < 4 || g + 1 < units) ? HALF : nmax - g * HALF; };

  // A scale too large for the pre-scaled route (any lane, any block): remembered, and acted on
  // once the loops are over; nothing is written before that. (Leaving the loop where the scale
  // is met costs every wave of the kernel: with that exit in it the compiler makes every wait
  // of the loop a wait for all loads in flight.)
  bool big = false;
  // the top of iteration blk (see above)
  auto block_top = [&](int blk) {
    big = stage_muls() || big;
    take_idx(blk + 1);
    issue_idx(blk + 2);
    stage_rows(blk + 1);
    lds_sync();
  };

  if (units > 0) {
    issue_idx(0);
    take_idx(0);
    issue_idx(1);
    stage_rows(0);
    lds_sync();
    // Iterations in which every unit exists and can be loaded run a copy of the loop without
    // conditions around its loads: the compiler places its waits by counting the loads behind
    // the one it waits for, and a load that may or may not have been issued counts as not
    // issued, which would turn every wait of the loop into a wait for everything.
    const bool steady = (loadable & 1u) != 0u && units >= 2;
    int blk = 0;
    if (steady) {
      if constexpr (HDRS_WITH_UNITS) issue_hdrs();
      issue_unit(raw_a, 0, HALF);
      issue_unit(raw_b, 1, HALF);
      const int steady_blocks = (units - 2) / U; // blocks whose last unit has two units behind it
      // (fp16 rows: and only blocks in which every entry adds a row; the first block with an
      // absent entry and all after it take the loop below, which clears what such entries load)
      for (; blk < steady_blocks && (QUANT || ((holey >> (blk & 1)) & 1u) == 0u); ++blk) {
        block_top(blk);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u & 1) {
            add_unit(raw_b, u, false, HALF);
            if (HDRS_WITH_UNITS && u + 2 == U) issue_hdrs();
            issue_unit(raw_b, blk * U + u + 2, HALF);
          } else {
            add_unit(raw_a, u, false, HALF);
            if (HDRS_WITH_UNITS && u + 2 == U) issue_hdrs();
            issue_unit(raw_a, blk * U + u + 2, HALF);
          }
          // units stay in this order: moved ahead of the arithmetic of earlier units, the loads
          // of later ones would need registers of their own
          __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_wave_barrier(); // the column lanes are done with the block before it is overwritten
      }
    } else {
      if constexpr (HDRS_WITH_UNITS) issue_hdrs();
      if (can_load(0)) issue_unit(raw_a, 0, live_rows(0));
      if (can_load(1)) issue_unit(raw_b, 1, live_rows(1));
    }
    for (; blk * U < units; ++blk) {
      block_top(blk);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int g = blk * U + u;
        if (g >= units) break; // no bag of the wave reaches this unit
        if (u & 1) {
          add_unit(raw_b, u, true, live_rows(g));
          if (HDRS_WITH_UNITS && u + 2 == U) issue_hdrs();
          if (can_load(g + 2)) issue_unit(raw_b, g + 2, live_rows(g + 2));
        } else {
          add_unit(raw_a, u, true, live_rows(g));
          if (HDRS_WITH_UNITS && u + 2 == U) issue_hdrs();
          if (can_load(g + 2)) issue_unit(raw_a, g + 2, live_rows(g + 2));
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if constexpr (QUANT) {
    if (__builtin_amdgcn_ballot_w64(big) != 0ull) return false; // wave-uniform
  }
  lean_report_bad(a, bad_pos);
  lean_write<EXACT, TY, C, INHDR, true, Q8>(a, d, L, table, acc, bsum, lds);
  return true;
}

// The same bags, one row at a time, integers converted to float before the fma:
// for waves that met a scale the pre-scaled arithmetic cannot take. Every lane
// walks its bag's entries itself; nothing is staged.
template <typename index_t, bool EXACT, int TY, int C, bool INHDR, bool Q8>
__device__ __forceinline__ void pool_lean_slow(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane, uint32_t* lds) {
  constexpr int E = TY == ST_INT4 ? 32 : 16;
  const LeanLane L = lean_lane<index_t>(a, d, table, first_slot, lane);
  const int S = d.lanes;
  const index_t* idx = reinterpret_cast<const index_t*>(a.indices) + L.pos0;
  const uint8_t* wbase = (d.placement ? a.weights[1] : a.weights[0]) + d.weights_offset;
  const int nchunks = INHDR ? (d.data_bytes + 4 + 15) / 16 : S * C;
  float acc[C * E];
#pragma unroll
  for (int e = 0; e < C * E; ++e) acc[e] = 0.0f;
  float bsum = -0.0f;
  int64_t bad_pos = LEAN_NO_BAD_POS;
  for (int i = 0; i < L.n; ++i) {
    int64_t row = (int64_t)idx[i];
    const float w = a.sample_weights ? a.sample_weights[L.pos0 + i] : 1.0f;
    if (L.remapped) row = lean_remap(a, L, row, L.pos0 + i, bad_pos);
    const int r = row == LEAN_PRUNED ? LEAN_SKIP : lean_row(d, L, row, L.pos0 + i, bad_pos);
    if (r < 0) continue;
    const uint8_t* prow = wbase + (uint64_t)(uint32_t)r * (uint32_t)d.row_stride;
    float rs, rb;
    load_scale_bias(prow + d.sb_off, d.sb_fp32 != 0, true, rs, rb);
    LeanMul m;
    m.s24 = w * rs;
    m.s20 = m.s24;
    m.bias = w * rb;
    m.hole = 0u;
    if constexpr (!EXACT) bsum += m.bias;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int k = L.sub + c * S;
      uint32_t raw[4];
      load_raw<16>(raw, prow + (INHDR ? 0 : d.data_off) + (k < nchunks ? k : nchunks - 1) * 16);
      lean_chunk<TY, EXACT, true, C * E>(acc, c * E, raw, m);
    }
  }
  lean_report_bad(a, bad_pos);
  lean_write<EXACT, TY, C, INHDR, false, Q8>(a, d, L, table, acc, bsum, lds);
}

template <typename index_t, bool EXACT, int TY, int C, bool INHDR, bool Q8>
__device__ __forceinline__ void run_lean(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane,
                                         uint32_t* lds) {
  bool done;
  if (d.lanes >= 8) done = pool_lean<index_t, EXACT, TY, C, INHDR, 1, Q8>(a, d, table, first_slot, lane, lds);
  else if (d.lanes >= 4) done = pool_lean<index_t, EXACT, TY, C, INHDR, 2, Q8>(a, d, table, first_slot, lane, lds);
  else done = pool_lean<index_t, EXACT, TY, C, INHDR, 4, Q8>(a, d, table, first_slot, lane, lds);
  if constexpr (TY == ST_INT4 || TY == ST_INT8) {
    if (!done) pool_lean_slow<index_t, EXACT, TY, C, INHDR, Q8>(a, d, table, first_slot, lane, lds);
  }
}

// Row types and the chunks per lane the host picks for lean shapes: 1 (4-bit), 2 (8-bit), 4 (fp16).
template <typename index_t, bool EXACT, bool Q8>
__device__ __forceinline__ void lean_dispatch(const LookupArgs& a, const TableDesc& d, int table, int first_slot, int lane,
                                              uint32_t* lds) {
  if (d.ty == ST_INT4) {
    if (d.inline_hdr) run_lean<index_t, EXACT, ST_INT4, 1, true, Q8>(a, d, table, first_slot, lane, lds);
    else run_lean<index_t, EXACT, ST_INT4, 1, false, Q8>(a, d, table, first_slot, lane, lds);
  } else if (d.ty == ST_INT8) {
    if (d.inline_hdr) run_lean<index_t, EXACT, ST_INT8, 2, true, Q8>(a, d, table, first_slot, lane, lds);
    else run_lean<index_t, EXACT, ST_INT8, 2, false, Q8>(a, d, table, first_slot, lane, lds);
  } else if (d.ty == ST_FP16) {
    run_lean<index_t, EXACT, ST_FP16, 4, false, Q8>(a, d, table, first_slot, lane, lds);
  }
}

#ifndef FBGEMM_AMD_LEAN_MIN_WAVES
#define FBGEMM_AMD_LEAN_MIN_WAVES 3 // waves per SIMD the register allocation must leave room for
#endif

// Same work list and workgroup -> XCD mapping as lookup_kernel. One wave per workgroup.
// Returns false when the workgroup has no work item.
__device__ __forceinline__ bool lean_work_item(const LookupArgs& a, int& table, int& first_slot) {
  int64_t wave;
  if (a.xcd_start) {
    const int xb = blockIdx.x & 7;
    const int64_t w = (int64_t)(blockIdx.x >> 3);
    const int64_t lo = a.xcd_start[xb], hi = a.xcd_start[xb + 1];
    if (w >= hi - lo) return false;
    wave = lo + w;
  } else {
    wave = (int64_t)blockIdx.x;
    if (wave >= a.num_waves) return false;
  }
  table = 0;
  if (a.work) {
    const WaveWork ww = a.work[wave];
    table = ww.table;
    first_slot = ww.first_bag;
  } else {
    first_slot = (int)(wave * a.single.bags);
  }
  return true;
}

template <typename index_t, bool EXACT, bool Q8>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(FBGEMM_AMD_LEAN_MIN_WAVES, 8))) void lookup_lean_kernel(const LookupArgs a) {
  // 8 KB: while a bag is pooled, two buffers of staged rows (2 KB) and the multipliers (4 KB); at the end, the wave's output
  __shared__ __attribute__((aligned(16))) uint32_t lds[LEAN_LDS_WORDS + MAX_GROUPS];
  int table, first_slot;
  if (!lean_work_item(a, table, first_slot)) return;
  const TableDesc d = a.tables ? a.tables[table] : a.single;
  lean_dispatch<index_t, EXACT, Q8>(a, d, table, first_slot, (int)threadIdx.x, lds);
}

// The instance for table-batched launches in which every table has 4-bit rows in bags of 8 lanes
// and more with the header fetched by a staging lane (lean_wide4_shape): that one instantiation
// of pool_lean (in the exact mode with units of 2 loads and the headers asked for at staging
// time, as in the kernel above; in the tolerance-grade mode with units of 4 and the headers next
// to their rows) needs 114 / 127 vector registers, so four waves fit a SIMD where the kernel
// above, which carries every row type and lane count, fits three. 16 instead of 12 waves per
// compute unit hide more of each other's waits: the HBM-sized configuration takes 14 % less in
// the exact mode and 8 % less in the tolerance-grade mode. (The table's descriptor is read from
// the device array only: the choice between that and the single-table descriptor of the
// launch arguments alone costs the registers that make the difference between 127 and a spill.)
// The rare path (a scale too large for the pre-scaled arithmetic) is not part of this kernel:
// inlined behind the common path it costs 30 registers more, and any spill makes every wave of
// the kernel reserve scratch memory. A wave that meets such a scale writes nothing and queues its
// work item; lookup_lean_wide4_redo_kernel, launched behind this kernel in every forward, pools
// the queued items with pool_lean_slow (usually none: 256 workgroups that read a zero and leave).
template <typename index_t, bool EXACT>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 8))) void lookup_lean_wide4_kernel(const LookupArgs a) {
  __shared__ __attribute__((aligned(16))) uint32_t lds[LEAN_LDS_WORDS + MAX_GROUPS];
  int table, first_slot;
  if (!lean_work_item(a, table, first_slot)) return;
  const TableDesc d = a.tables[table]; // table-batched launches only
  const int lane = (int)threadIdx.x;
  const bool done = pool_lean<index_t, EXACT, ST_INT4, 1, false, 1, false, EXACT ? 2 : 4, EXACT>(a, d, table, first_slot, lane, lds);
  if (!done && lane == 0) { // wave-uniform verdict; nothing has been written or reported
    const int k = atomicAdd(a.redo_count, 1);
    WaveWork ww;
    ww.table = table;
    ww.first_bag = first_slot;
    a.redo[k] = ww;
  }
}

constexpr int LEAN_REDO_WORKGROUPS = 256;
template <typename index_t, bool EXACT>
__global__ __launch_bounds__(64) void lookup_lean_wide4_redo_kernel(const LookupArgs a) {
  __shared__ __attribute__((aligned(16))) uint32_t lds[LEAN_LDS_WORDS + MAX_GROUPS];
  const int lane = (int)threadIdx.x;
  const int count = __hip_atomic_load(a.redo_count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // the ticket is taken once the count has arrived (its increment depends on it): whoever draws the
  // last ticket knows that every workgroup of the launch holds its copy of the count
  int ticket = 0;
  if (lane == 0) ticket = atomicAdd(a.redo_count + 1, count >= 0 ? 1 : 2);
  ticket = __builtin_amdgcn_readfirstlane(ticket);
  for (int i = (int)blockIdx.x; i < count; i += (int)gridDim.x) {
    const WaveWork ww = a.redo[i];
    const TableDesc d = a.tables ? a.tables[ww.table] : a.single;
    pool_lean_slow<index_t, EXACT, ST_INT4, 1, false, false>(a, d, ww.table, ww.first_bag, lane, lds);
  }
  if (ticket == (int)gridDim.x - 1 && lane == 0) { // for the next forward
    a.redo_count[0] = 0;
    a.redo_count[1] = 0;
  }
}

#define FBGEMM_AMD_DEFINE_LEAN_LAUNCH(FN, INDEX_T, EXACT, Q8)                                            \
  hipError_t FN(const LookupArgs& a, unsigned blocks, hipStream_t stream) {                              \
    hipLaunchKernelGGL((lookup_lean_kernel<INDEX_T, EXACT, Q8>), dim3(blocks), dim3(64), 0, stream, a);  \
    return hipGetLastError();                                                                            \
  }

#define FBGEMM_AMD_DEFINE_LEAN_WIDE4_LAUNCH(FN, INDEX_T, EXACT)                                           \
  hipError_t FN(const LookupArgs& a, unsigned blocks, hipStream_t stream) {                              \
    hipLaunchKernelGGL((lookup_lean_wide4_kernel<INDEX_T, EXACT>), dim3(blocks), dim3(64), 0, stream, a); \
    hipLaunchKernelGGL((lookup_lean_wide4_redo_kernel<INDEX_T, EXACT>), dim3(LEAN_REDO_WORKGROUPS), dim3(64), 0, stream, a); \
    return hipGetLastError();                                                                            \
  }

} // namespace fbgemm_amd
