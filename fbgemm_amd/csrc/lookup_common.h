// Shared between the host-side launch code and the gfx950 kernels.
#pragma once
#include <stdint.h>

namespace fbgemm_amd {

// Row element types, numbered like the reference's SparseType
// (fbgemm_gpu/include/fbgemm_gpu/embedding_common.h:20-32).
enum : int32_t {
  ST_FP32 = 0,
  ST_FP16 = 1,
  ST_INT8 = 2,
  ST_INT4 = 3,
  ST_INT2 = 4,
  ST_BF16 = 5,
  ST_FP8 = 6, // 8-bit floats (1 sign, e exponent, 7 - e mantissa bits; exponent bias given per call)
};

// Bits of the status word a lookup ORs in when it meets an input the reference
// would reject (src/RefImplementations.cc:1294-1306,1346).
enum : int32_t {
  ERR_INDEX_OUT_OF_RANGE = 1, // idx < 0 (and not a skipped -1) or idx >= rows
  ERR_BAG_OVERRUN = 2,        // a bag ends past index_size / past the index array
  ERR_LENGTH_MISMATCH = 4,    // sum of bag lengths != index_size
  ERR_NEGATIVE_LENGTH = 8,    // offsets decrease (the reference's result is then undefined)
};

// Device status block: word 0 = OR of ERR_* bits, words 2..3 = the smallest
// position (into the index array) of an out-of-range index, as an int64
// minimum so that the first offender in index order wins deterministically.
struct Status {
  int32_t bits;
  int32_t pad;
  unsigned long long first_bad_pos;
};

// How a wave walks one table. Filled on the host from the table's element
// type, dimension, stride and alignment.
struct TableDesc {
  int64_t weights_offset; // byte offset of row 0 inside the weights buffer
  int64_t row_stride;     // bytes between consecutive rows
  int64_t num_rows;       // exclusive bound for a valid physical row id
  int32_t D;              // elements per row
  int32_t out_col;        // first output column of this table's block
  int32_t ty;             // ST_*
  int32_t vb;             // bytes each lane loads per row and pass: 1, 2, 4 or 16
  int32_t sb_off;         // byte offset of (scale, bias) inside a row
  int32_t data_off;       // byte offset of the element data inside a row
  int32_t sb_fp32;        // 1: scale/bias are two floats, 0: two halfs
  int32_t lanes;          // lanes cooperating on one bag (1..64)
  int32_t passes;         // column passes when a row exceeds lanes * vb bytes
  int32_t placement;      // which of the two weights buffers holds the table
  int32_t data_bytes;     // bytes of element data per row (unpadded)
  int32_t skip_minus_one; // 1: an index of -1 is a pruned row and is skipped
  int32_t vec_store;      // bit 0 / bit 1: every lane's output run is aligned for whole-run
                          // vector stores with 4-byte / 2-byte output elements
  int32_t chunks;         // 16-byte chunks per lane and pass (1, 2 or 4)
  int32_t inline_hdr;     // 1: lanes own 16-byte chunks of the WHOLE row (fp16 scale/bias
                          // header first, then data), so the header arrives with the data
                          // and costs no request of its own; `lanes` need not divide 64
  int32_t packed;         // 1: bags lie end to end in the wave (see bags_per_wave)
  int32_t lanes_recip;    // ceil(65536 / lanes): j / lanes == (j * lanes_recip) >> 16 for 0 <= j <= 64
  int32_t bags;           // bags_per_wave(lanes, packed), so that no kernel divides
};

#if defined(__HIPCC__)
// Streaming stores for output a kernel never reads back: marked non-temporal so
// that the lines do not displace table rows and indices in the caches. Same
// bytes as a plain store of the same width; `p` must be aligned to the width.
typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t stream_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stream_store16(void* p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const stream_u32x4 q = {a, b, c, d};
  __builtin_nontemporal_store(q, reinterpret_cast<stream_u32x4*>(p));
}
__device__ __forceinline__ void stream_store16(void* p, float a, float b, float c, float d) {
  stream_store16(p, __float_as_uint(a), __float_as_uint(b), __float_as_uint(c), __float_as_uint(d));
}
__device__ __forceinline__ void stream_store8(void* p, uint32_t a, uint32_t b) {
  const stream_u32x2 q = {a, b};
  __builtin_nontemporal_store(q, reinterpret_cast<stream_u32x2*>(p));
}
__device__ __forceinline__ void stream_store4(void* p, uint32_t a) {
  __builtin_nontemporal_store(a, reinterpret_cast<uint32_t*>(p));
}
#endif

// Bags a wave pools side by side when `lanes` lanes share a bag. The memory
// pipeline merges the addresses of a 16-byte-per-lane load 16 lanes at a time,
// so a bag's lanes should not straddle a multiple of 16: with `packed` = 0 each
// quarter of the wave holds 16 / lanes whole bags and leaves the rest of its
// lanes idle (for the powers of two this is 64 / lanes). Where that would idle
// too many lanes (9 lanes per bag: 7 of every 16), `packed` = 1 lays the bags
// end to end instead: 64 / lanes bags, some of which straddle a quarter and
// cost an extra line request now and then.
#if defined(__HIPCC__)
__host__ __device__
#endif
inline int bags_per_wave(int lanes, int packed) { return (lanes <= 16 && !packed) ? 4 * (16 / lanes) : 64 / lanes; }

// What the bag scheduler leaves per bag, in the order waves take the bags.
struct __attribute__((aligned(16))) BagEntry {
  int64_t o0;  // offsets[bag]
  int32_t len; // offsets[bag + 1] - offsets[bag]; -1 when that is negative or beyond 31 bits: the
               // lookup then reads the two offsets itself and reports what it finds
  int32_t bag; // bag id inside its table
};

// The pruned-row mapping of an order-preserving table, 32 logical rows per record
// (remap_rank_kernels.hip): physical row = before + popcount(bits below the row's bit).
struct __attribute__((aligned(8))) RankRecord {
  uint32_t before; // kept rows in front of the record's first logical row
  uint32_t bits;   // bit b: logical row 32 * record + b is kept
};

// One entry per wave: which table and which first position of the bag order.
struct WaveWork {
  int32_t table;
  int32_t first_bag;
};

struct LookupArgs {
  const TableDesc* tables;   // device array, or nullptr when `single` is used
  TableDesc single;
  const uint8_t* weights[2]; // buffers selected by TableDesc::placement
  const void* indices;
  const void* offsets;       // T*B+1 offsets ((table, bag) order)
  const float* sample_weights; // nullptr: unweighted
  const void* remap;         // logical -> physical row table(s), int32 or int64, or nullptr
  const int64_t* remap_offsets; // nullptr: one table of remap_rows entries; else T+1 offsets
                             // into `remap`, an empty range meaning "this table is not pruned"
  int64_t remap_rows;        // bound for logical ids when remap_offsets == nullptr
  int32_t remap64;           // remap entries are int64 (else int32)
  const RankRecord* rank_records; // nullptr, or the compact form of the mappings of order-preserving tables
  const int64_t* rank_offsets;    // T entries: first record of table t, or -1: the table's mapping is read from `remap`
  void* out;
  int64_t out_stride;        // elements between consecutive bags' outputs
  int64_t index_size;        // entries the index array holds for this call
  const BagEntry* order;     // per table, its B bags in the order waves take them
                             // (longest first), or nullptr: natural order
  const WaveWork* work;      // per-wave work list, or nullptr: single table, dense mapping
  const int64_t* xcd_start;  // 9 entries: the work list is 8 runs, run x = [xcd_start[x],
                             // xcd_start[x+1]) is walked by the workgroups with id % 8 == x
                             // (the workgroups one XCD receives); nullptr: one run
  int64_t num_waves;         // waves with work (longest run when xcd_start is used)
  int32_t B;                 // bags per table
  int32_t T;
  int32_t out_ty;            // ST_FP32, ST_FP16 or ST_BF16; the lean kernel also takes ST_INT8 (lean_store_q8: `out` is bytes,
                             // out_stride bytes per line, table t's block 8 t bytes behind its column)
  int32_t off64;             // offsets are int64 (else int32)
  int32_t normalize;         // mean pooling: scale by 1/len, len counting skipped rows
  int32_t positional;        // weight of entry i of a bag is sample_weights[i]
  int32_t check_total;       // single-table call: positions are relative to offsets[0] and
                             // offsets[last] - offsets[0] must equal index_size
  int32_t out_aligned;       // `out` is 16-byte aligned (vector stores allowed)
  int32_t fp8_shift;         // FP8 rows: 16 + exponent bits (moves the 7 low bits to fp32's exponent/mantissa)
  float fp8_mult;            // FP8 rows: 2^(127 - exponent bias)
  // lookup_lean_wide4_kernel only: where a wave that meets a scale too large for its arithmetic
  // leaves its work item (redo[atomicAdd(redo_count, 1)]) for lookup_lean_wide4_redo_kernel, which
  // pools those items the plain way afterwards. redo_count[1] counts that kernel's workgroups; its
  // last one sets both counters back to zero.
  WaveWork* redo;
  int32_t* redo_count;
  Status* status;
};

} // namespace fbgemm_amd
