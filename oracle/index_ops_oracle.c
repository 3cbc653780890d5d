/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the index operators that run before
 * the quantized embedding-bag lookup: bounds_check_indices and the pruned-row
 * hash map (insert, lookup).
 *
 * A plain-C restatement of the reference's CPU operators, loop for loop (the
 * order of the loops matters: a bag whose offsets are repaired changes what the
 * next bag reads). Nothing in the shipped library links, loads or calls this
 * file.
 *
 * Parity status: PINNED. tests/test_index_ops_oracle.py checks
 *   - the properties the reference's own test asserts
 *     (fbgemm_gpu/test/tbe/utils/split_embeddings_utils_test.py:237-465: inputs
 *     in bounds are left alone; all-out-of-range indices become 0 and are counted
 *     one by one; offsets[0] = -100 and offsets[-1] += 100 are repaired to 0 and
 *     to the number of indices; FATAL reports instead of repairing),
 *   - the closed form of the repaired offsets (running maximum of the offsets
 *     clamped to [0, num_indices]),
 *   - the hash functions against the published MurmurHash3 finalizers' known
 *     answers (fmix32 / fmix64) and the map against a Python dict (every
 *     inserted key is found with its value, every other key gives -1),
 *     including colliding keys and a wrapped probe sequence;
 * tests/test_prune_oracle.py checks oracle_rowwise_prune against
 * torch._rowwise_prune (the ATen routine the reference's operator ends in) and
 * its keep rule by brute force over short inputs.
 *
 * Reference files followed:
 *   fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:48-219
 *   fbgemm_gpu/codegen/inference/embedding_forward_quantized_cpu_template.cpp:102-204
 *                                        (hash functions, pruned_hashmap_insert)
 *   fbgemm_gpu/codegen/inference/embedding_forward_quantized_cpu_template.cpp:524-603
 *                                        (pruned_hashmap_lookup)
 *   fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2836-2893  embedding_bag_rowwise_prune
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static int64_t rd(const void* p, int is64, int64_t i) {
  return is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}
static void wr(void* p, int is64, int64_t i, int64_t v) {
  if (is64) ((int64_t*)p)[i] = v;
  else ((int32_t*)p)[i] = (int32_t)v;
}

enum { MODE_FATAL = 0, MODE_WARNING = 1, MODE_IGNORE = 2 };
/* what a FATAL run reports (same bits as the library's status word) */
enum { ERR_INDEX_OUT_OF_RANGE = 1, ERR_BAG_OVERRUN = 2, ERR_LENGTH_MISMATCH = 4 };

/* embedding_bounds_check_host_cpu.cpp:48-62 */
static void adjust_offset(int64_t* start, int64_t* end, int64_t num_indices) {
  int64_t s = *start, e = *end;
  s = s < num_indices ? s : num_indices;
  s = s > 0 ? s : 0;
  e = e < num_indices ? e : num_indices;
  e = e > s ? e : s;
  *start = s;
  *end = e;
}

/*
 * bounds_check_indices_cpu (embedding_bounds_check_host_cpu.cpp:76-219).
 * indices / offsets are modified in place (WARNING, IGNORE); `warning` is the
 * one-element counter tensor (zeroed first in WARNING mode, :103-105).
 * B_offsets == NULL: every table has B = (offsets_numel - 1) / T bags.
 * Returns 0, or in FATAL mode the OR of the ERR_* conditions of the FIRST check
 * that would have raised (the reference stops there; nothing is modified).
 */
int oracle_bounds_check_indices(
    const int64_t* rows_per_table, int32_t T, void* indices, void* offsets, int idx64,
    int64_t num_indices, int64_t offsets_numel, int mode, int64_t* warning,
    const int32_t* B_offsets) {
  const int64_t total_B = offsets_numel - 1;
  const int64_t B = T > 0 ? total_B / T : 0;
  if (mode == MODE_WARNING) warning[0] = 0;
  if (mode == MODE_FATAL) {
    if (num_indices != rd(offsets, idx64, total_B)) return ERR_LENGTH_MISMATCH;
  } else if (num_indices != rd(offsets, idx64, total_B)) {
    if (mode == MODE_WARNING) warning[0] += 1;
    wr(offsets, idx64, total_B, num_indices);
  }
  for (int32_t t = 0; t < T; ++t) {
    const int64_t num_rows = rows_per_table[t];
    const int64_t B_begin = B_offsets ? B_offsets[t] : t * B;
    const int64_t B_end = B_offsets ? B_offsets[t + 1] : (t + 1) * B;
    for (int64_t b = 0; b < B_end - B_begin; ++b) {
      int64_t start = rd(offsets, idx64, B_begin + b);
      int64_t end = rd(offsets, idx64, B_begin + b + 1);
      const int bad = start < 0 || start > end || end > num_indices;
      if (mode == MODE_FATAL) {
        if (bad) return ERR_BAG_OVERRUN;
      } else if (mode == MODE_IGNORE || bad) {
        if (mode == MODE_WARNING) warning[0] += 1;
        adjust_offset(&start, &end, num_indices);
        wr(offsets, idx64, B_begin + b, start);
        wr(offsets, idx64, B_begin + b + 1, end);
      }
      for (int64_t l = 0; l < end - start; ++l) {
        const int64_t idx = rd(indices, idx64, start + l);
        if (idx == -1) continue; /* pruned row */
        if (idx < 0 || idx >= num_rows) {
          if (mode == MODE_FATAL) return ERR_INDEX_OUT_OF_RANGE;
          if (mode == MODE_WARNING) warning[0] += 1;
          wr(indices, idx64, start + l, 0);
        }
      }
    }
  }
  return 0;
}

/* MurmurHash3 finalizers (embedding_forward_quantized_cpu_template.cpp:102-120) */
uint32_t oracle_pruned_hash32(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}
uint64_t oracle_pruned_hash64(uint64_t k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return k;
}

/* first slot of a key: the index width picks the hash (…cpu_template.cpp:146-147,175) */
static int64_t first_slot(int64_t idx, int idx64, int64_t capacity) {
  if (idx64) return (int64_t)(oracle_pruned_hash64((uint64_t)idx) % (uint64_t)capacity);
  return (int64_t)((int64_t)oracle_pruned_hash32((uint32_t)(int32_t)idx) % capacity);
}

/*
 * pruned_hashmap_insert (…cpu_template.cpp:123-204). hash_table: [slots][2]
 * of int32 or int64 (key, value), empty = -1. A full table with a new key would
 * probe forever in the reference; here the call returns -1 instead.
 */
int oracle_pruned_hashmap_insert(
    int32_t T, int32_t B, const void* indices, const void* dense_indices, const void* offsets,
    int idx64, void* hash_table, int hash64, const int64_t* hash_table_offsets) {
  for (int32_t t = 0; t < T; ++t) {
    const int64_t table_start = hash_table_offsets[t];
    const int64_t capacity = hash_table_offsets[t + 1] - table_start;
    if (capacity == 0) continue;
    for (int32_t b = 0; b < B; ++b) {
      const int64_t s = rd(offsets, idx64, (int64_t)t * B + b);
      const int64_t e = rd(offsets, idx64, (int64_t)t * B + b + 1);
      for (int64_t i = s; i < e; ++i) {
        const int64_t idx = rd(indices, idx64, i);
        const int64_t dense = rd(dense_indices, idx64, i);
        if (dense == -1) continue;
        int64_t slot = first_slot(idx, idx64, capacity);
        int64_t probes = 0;
        for (;; ++probes) {
          if (probes > capacity) return -1;
          const int64_t at = table_start + slot;
          const int64_t key = rd(hash_table, hash64, 2 * at);
          if (key == -1) {
            wr(hash_table, hash64, 2 * at, idx);
            wr(hash_table, hash64, 2 * at + 1, dense);
            break;
          }
          if (key == idx) {
            wr(hash_table, hash64, 2 * at + 1, dense);
            break;
          }
          slot = (slot + 1) % capacity;
        }
      }
    }
  }
  return 0;
}

/* pruned_hashmap_lookup (…cpu_template.cpp:524-603); a key that is absent from a
 * table without an empty slot gives -1 after one trip round the table */
void oracle_pruned_hashmap_lookup(
    int32_t T, int32_t B, const void* indices, const void* offsets, int idx64,
    const void* hash_table, int hash64, const int64_t* hash_table_offsets, void* dense_indices) {
  for (int32_t t = 0; t < T; ++t) {
    const int64_t table_start = hash_table_offsets[t];
    const int64_t capacity = hash_table_offsets[t + 1] - table_start;
    const int64_t s = rd(offsets, idx64, (int64_t)t * B);
    const int64_t e = rd(offsets, idx64, (int64_t)(t + 1) * B);
    for (int64_t i = s; i < e; ++i) {
      const int64_t idx = rd(indices, idx64, i);
      if (capacity == 0) {
        wr(dense_indices, idx64, i, idx);
        continue;
      }
      int64_t slot = first_slot(idx, idx64, capacity);
      int64_t out = -1;
      for (int64_t probes = 0; probes < capacity; ++probes) {
        const int64_t at = table_start + slot;
        const int64_t key = rd(hash_table, hash64, 2 * at);
        if (key == -1) break;
        if (key == idx) {
          out = rd(hash_table, hash64, 2 * at + 1);
          break;
        }
        slot = (slot + 1) % capacity;
      }
      wr(dense_indices, idx64, i, out);
    }
  }
}

/* ---- embedding_bag_rowwise_prune ---------------------------------------------
 * fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2836-2893: the sequential loop that
 * decides which rows stay (indicator above the threshold, compared in double; once
 * the rows kept so far plus all rows still to come do not exceed
 * min_non_pruned_rows, every remaining row stays), followed by what
 * at::native::_rowwise_prune does with that mask: kept rows are copied in order,
 * remap[i] is the new row id or -1. Returns the number of rows kept; out_weights
 * may be NULL (mask and remap only). Pinned by tests/test_prune_oracle.py against
 * torch._rowwise_prune (the ATen routine the reference calls) and by brute force
 * over all masks of short inputs. */
int64_t oracle_rowwise_prune(const float* weights, const float* indicator, int64_t rows, int64_t cols, double threshold,
                             int use_abs, int64_t min_non_pruned_rows, int idx64, void* remap, float* out_weights) {
  int64_t num_kept = 0;
  for (int64_t i = 0; i < rows; ++i) {
    const float val = use_abs ? fabsf(indicator[i]) : indicator[i];
    int keep = (double)val > threshold;
    if (num_kept < min_non_pruned_rows && num_kept + (rows - i) <= min_non_pruned_rows) keep = 1;
    const int64_t id = keep ? num_kept : -1;
    if (idx64) ((int64_t*)remap)[i] = id;
    else ((int32_t*)remap)[i] = (int32_t)id;
    if (!keep) continue;
    if (out_weights) memcpy(out_weights + num_kept * cols, weights + i * cols, sizeof(float) * (size_t)cols);
    ++num_kept;
  }
  return num_kept;
}
