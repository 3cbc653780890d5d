// The general pooled-lookup kernel: any row type, width, alignment and option
// of the single-table and table-batched entry points. Included by one
// translation unit per (index type, GENERAL) instance so that they compile
// side by side.
#pragma once
#include "lookup_device.h"

namespace fbgemm_amd {

// ---- one wave, one table ----------------------------------------------------



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
  const int G = d.bags;
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
      o1 = o0 + be.len;
      if (be.len < 0) { // a length the entry cannot hold: judge the offsets themselves
        o0 = read_offset(a.offsets, a.off64, ob + be.bag);
        o1 = read_offset(a.offsets, a.off64, ob + be.bag + 1);
      }
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
  int64_t remap_base = 0, remap_cap = 0, rank_base = -1;
  bool remapped = false;
  if (GENERAL && a.remap) {
    remapped = true;
    remap_cap = a.remap_rows;
    if (a.remap_offsets) {
      remap_base = a.remap_offsets[table];
      remap_cap = a.remap_offsets[table + 1] - remap_base;
      remapped = remap_cap > 0;
      if (a.rank_records) rank_base = a.rank_offsets[table];
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
              if (rank_base >= 0) { // order-preserving mapping: the rank among the kept rows (remap_rank_kernels.hip)
                const RankRecord rr = a.rank_records[rank_base + (row >> 5)];
                const uint32_t bit = (uint32_t)row & 31u;
                row = ((rr.bits >> bit) & 1u) ? (int64_t)(rr.before + (uint32_t)__builtin_popcount(rr.bits & ((1u << bit) - 1u))) : -1;
              } else {
                row = a.remap64 ? reinterpret_cast<const int64_t*>(a.remap)[remap_base + row]
                                : (int64_t) reinterpret_cast<const int32_t*>(a.remap)[remap_base + row];
              }
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
    first_slot = (int)(wave * a.single.bags);
  }
  const TableDesc d = a.tables ? a.tables[table] : a.single;
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
}


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
  run_item<index_t, GENERAL>(a, wave, lane, stage_row, stage_mul);
}


// Defines the launcher of one instance of lookup_kernel.
#define FBGEMM_AMD_DEFINE_LOOKUP_LAUNCH(FN, INDEX_T, GENERAL)                                             \
  hipError_t FN(const LookupArgs& a, unsigned blocks, hipStream_t stream) {                              \
    hipLaunchKernelGGL((lookup_kernel<INDEX_T, GENERAL>), dim3(blocks), dim3(64), 0, stream, a);         \
    return hipGetLastError();                                                                            \
  }

} // namespace fbgemm_amd
