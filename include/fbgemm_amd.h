/*
 * fbgemm_amd -- C ABI of the MI355X (gfx950) quantized embedding-bag library.
 *
 * Every data pointer named d_* is a DEVICE pointer (HBM). `stream` is a
 * hipStream_t passed as void* (NULL = the default stream). Launch calls are
 * asynchronous: they enqueue on `stream` and return. Nothing is allocated per
 * call except where a function says so.
 *
 * Return values: 0 = enqueued / done, < 0 = FBGEMM_AMD_E_* (bad argument or a
 * HIP error). Input errors that the reference reports by returning false
 * (index out of range, bag overrun, length mismatch) are detected ON THE
 * DEVICE and recorded in a 16-byte status block the caller owns; read it back
 * with fbgemm_amd_status_read (this is the only call that synchronizes).
 */
#ifndef FBGEMM_AMD_H_
#define FBGEMM_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types; values follow the reference's SparseType
 * (fbgemm_gpu/include/fbgemm_gpu/embedding_common.h:20-32). */
enum {
  FBGEMM_AMD_FP32 = 0,
  FBGEMM_AMD_FP16 = 1,
  FBGEMM_AMD_INT8 = 2,
  FBGEMM_AMD_INT4 = 3,
  FBGEMM_AMD_INT2 = 4,
  FBGEMM_AMD_BF16 = 5,
  FBGEMM_AMD_FP8 = 6
};

/* Pooling modes (embedding_common.h:34). NONE (one output row per index) has its own entry point,
 * fbgemm_amd_tbe_forward_nobag. */
enum { FBGEMM_AMD_POOL_SUM = 0, FBGEMM_AMD_POOL_MEAN = 1, FBGEMM_AMD_POOL_NONE = 2 };

/* Error codes returned by the entry points. */
enum {
  FBGEMM_AMD_OK = 0,
  FBGEMM_AMD_E_ARG = -1,      /* invalid argument combination */
  FBGEMM_AMD_E_HIP = -2,      /* a HIP runtime call failed; see fbgemm_amd_last_error */
  FBGEMM_AMD_E_UNSUPPORTED = -3
};

/* Bits of the device status word (what made the reference return false). */
enum {
  FBGEMM_AMD_ERR_INDEX_OUT_OF_RANGE = 1,
  FBGEMM_AMD_ERR_BAG_OVERRUN = 2,
  FBGEMM_AMD_ERR_LENGTH_MISMATCH = 4,
  FBGEMM_AMD_ERR_NEGATIVE_LENGTH = 8
};

#define FBGEMM_AMD_STATUS_BYTES 16

/* Human-readable text of the last FBGEMM_AMD_E_* on this thread. */
const char* fbgemm_amd_last_error(void);

/* Library version, "major.minor". */
const char* fbgemm_amd_version(void);

/* ---- status block ------------------------------------------------------- */

/* Reset a status block (launches a one-thread fill kernel; capture-safe). */
int fbgemm_amd_status_clear(void* d_status, void* stream);

/* Synchronize `stream`, copy the block back. *bits = OR of FBGEMM_AMD_ERR_*;
 * *first_bad_pos = smallest position in the index array holding an
 * out-of-range index, or -1. Either out pointer may be NULL. */
int fbgemm_amd_status_read(const void* d_status, void* stream, int32_t* bits, int64_t* first_bad_pos);

/* ---- single-table pooled lookup ----------------------------------------- *
 *
 * Replaces the kernels returned by fbgemm::GenerateEmbeddingSpMDMWithStrides,
 * GenerateEmbeddingSpMDMNBitWithStrides, GenerateEmbeddingSpMDMFP8WithStrides,
 * GenerateEmbeddingSpMDMRowWiseSparse and GenerateEmbeddingSpMDMNBitRowWiseSparse
 * (include/fbgemm/FbgemmEmbedding.h:94-117,151-174,185-203,229-262): the config holds
 * what those factories fix at generation time, the launch takes what
 * EmbeddingSpMDMKernelSignature::Type takes (FbgemmEmbedding.h:41-49,211-221).
 */
typedef struct fbgemm_amd_spmdm_config {
  int32_t weight_ty;            /* FBGEMM_AMD_INT8/INT4/INT2/FP16/BF16/FP32/FP8 */
  int32_t output_ty;            /* FBGEMM_AMD_FP32/FP16/BF16 (no_bag: also INT8/INT4) */
  int32_t index_bits;           /* 32 or 64 */
  int32_t offset_bits;          /* 32 or 64 */
  int64_t block_size;           /* elements per row (D) */
  int64_t output_stride;        /* elements between output rows; -1 = block_size */
  int64_t input_stride;         /* storage elements between table rows (bytes for the
                                   integer formats, halfs for fp16/bf16, floats for
                                   fp32); -1 = densely packed rows */
  int32_t normalize_by_lengths; /* mean pooling */
  int32_t is_weight_positional; /* weights[i] belongs to entry i of every bag */
  int32_t use_offsets;          /* 1: offsets[output_size+1]; 0: lengths[output_size] */
  int32_t scale_bias_last;      /* 1: scale/bias after the row data (fp32 pair for
                                   INT8, fp16 pair for INT4/INT2); 0: fp16 pair in
                                   front of the data, and index -1 is skipped */
  int32_t no_bag;               /* 1: no pooling, one output row per index (the
                                   factories' no_bag flag, FbgemmEmbedding.h:113,170;
                                   src/RefImplementations.cc:1235-1288,1352-1376,
                                   1466-1484): output_size indices, offsets unused,
                                   d_weights[m] scales row m, -1 is out of range.
                                   output_ty INT8 (8-bit rows) copies the first
                                   min(output_stride, input_stride) bytes of each row
                                   to rows output_stride bytes apart; output_ty INT4
                                   (4-bit rows, the only output they have) copies
                                   input_stride bytes to rows input_stride apart */
  int32_t fp8_exponent_bits;    /* weight_ty FP8 (GenerateEmbeddingSpMDMFP8WithStrides, */
  int32_t fp8_exponent_bias;    /* FbgemmEmbedding.h:185-203): the format of the rows */
  int32_t accumulate;           /* FBGEMM_AMD_ACC_EXACT (0, the default) or
                                   FBGEMM_AMD_ACC_FAST, see below */
} fbgemm_amd_spmdm_config;

/* How 4- and 8-bit rows are accumulated. No counterpart in the reference.
 * EXACT: the reference's own sequence of fp32 roundings, acc = fma(scale, q,
 *   acc + bias) per element in index order (src/RefImplementations.cc:1326-1333,
 *   1519-1527): results are bit-identical to the CPU path.
 * FAST: the biases of a bag are summed apart, acc = fma(scale, q, acc) per
 *   element, out = acc + sum of the biases: a third fewer vector instructions
 *   per 4-bit element. Same index order, one lane per output column, so results
 *   are deterministic and differ from the reference's by a few fp32 roundings of
 *   the partial sums (tests hold every element that is not a cancellation to
 *   1e-5 relative for fp32 output and to one unit in the last place of fp16 /
 *   bf16 output). A call of few, long bags (fewer than 256 waves, 32 rows per
 *   bag and more) over such rows is cut into segments whose fp32 partial sums
 *   are added in order afterwards: still deterministic, another association of
 *   the same sum.
 * Only 4- and 8-bit rows of the regular shapes (whole 16-byte chunks, 32
 * columns per lane) have the FAST arithmetic; 4- and 8-bit rows of other widths
 * are summed the EXACT way inside a segment but may still be cut into segments.
 * 2-bit, fp16 / bf16 / fp32 / fp8 rows are computed the EXACT way in either
 * mode and never in segments: a table-batched plan cuts bags only when every
 * one of its tables has 4- or 8-bit rows. */
enum { FBGEMM_AMD_ACC_EXACT = 0, FBGEMM_AMD_ACC_FAST = 1 };

/* Enqueue one pooled lookup. d_weights may be NULL (unweighted).
 * d_compressed_indices_table, when non-NULL, selects the row-wise-sparse
 * variant: data_size then bounds the LOGICAL ids and the table maps them to
 * physical rows (-1 = pruned). d_status must be a cleared status block.
 * With use_offsets == 0 the call makes a prefix sum of the lengths into a
 * library-owned scratch buffer first (grown with hipMalloc when too small).
 * The library keeps one set of scratch buffers (and one status block for
 * fbgemm_amd_spmdm_run) per host thread and device: host threads may call
 * concurrently, each on its own stream; the calls of one thread that use
 * scratch must be ordered on one stream. */
int fbgemm_amd_spmdm_launch(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_compressed_indices_table, void* d_status, void* stream);

/* fbgemm_amd_spmdm_launch for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. Same arguments, same
 * kernels; the same results bit for bit with FBGEMM_AMD_ACC_EXACT, and with
 * FBGEMM_AMD_ACC_FAST whenever the call above does not cut the bags into
 * segments (this entry point never does: the segments' partial sums need
 * scratch of a size it has no place for). The two pieces of scratch the call above
 * takes from hipMalloc'ed buffers (the prefix sum of the lengths when
 * use_offsets == 0, and the bag order of the scheduler for calls of 2^21
 * lookups and more) live in a static device array of the library instead
 * (about 1.5 MiB, held by every GPU the library runs on until the process
 * ends). Limit: output_size <= FBGEMM_AMD_NOALLOC_MAX_BAGS, larger calls are
 * rejected with FBGEMM_AMD_E_ARG. It calls no hipMalloc / hipFree and no
 * allocating library routine; its first call on a device asks the runtime for
 * the array's device address (no allocation, but make that call outside a
 * graph capture). All calls on one GPU share the array: two of them that
 * overlap in time (different streams, or host threads without ordering) race;
 * order them on one stream. Nothing in the array has to start at zero (every
 * call writes what it reads). */
#define FBGEMM_AMD_NOALLOC_MAX_BAGS 65536
int fbgemm_amd_spmdm_launch_noalloc(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_compressed_indices_table, void* d_status, void* stream);
/* The limit above, for callers that bind the library without its header. */
int64_t fbgemm_amd_noalloc_max_bags(void);

/* Same, synchronous, with the reference's return convention: 1 = true,
 * 0 = false (the inputs were rejected; output unspecified), < 0 = API error.
 * Uses a library-owned status block. */
int fbgemm_amd_spmdm_run(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_compressed_indices_table, void* stream);

/* ---- table-batched forward ----------------------------------------------- *
 *
 * Replaces int_nbit_split_embedding_codegen_lookup_function
 * (fbgemm_gpu/codegen/inference/embedding_forward_quantized_host_cpu.cpp:84-227,
 * embedding_forward_quantized_cpu_template.cpp:208-520; GPU dispatcher
 * embedding_forward_quantized_host.cpp:259-370). A plan is made once from the
 * operator's metadata tensors (HOST copies), then reused for every forward.
 */
typedef struct fbgemm_amd_tbe_plan fbgemm_amd_tbe_plan;

/* weights_offsets[T] (bytes), weights_tys[T] (element types), D_offsets[T+1],
 * weights_placements[T] (0 = dev_weights, anything else = uvm_weights) are the
 * operator's tensors of the same names, on the host. *_weights_bytes are the
 * sizes of the two weights buffers (they bound the last table's row count, as
 * embedding_forward_quantized_cpu_template.cpp:372-380 does). row_alignment
 * is the operator's argument (16 on GPU builds of the reference). */
int fbgemm_amd_tbe_plan_create(
    fbgemm_amd_tbe_plan** plan, int32_t T, const int64_t* weights_offsets,
    const uint8_t* weights_tys, const int32_t* D_offsets,
    const int32_t* weights_placements, int64_t dev_weights_bytes,
    int64_t uvm_weights_bytes, int64_t row_alignment);

void fbgemm_amd_tbe_plan_destroy(fbgemm_amd_tbe_plan* plan);

/* Enqueue the forward of all T tables in ONE kernel launch.
 * d_offsets holds T*B+1 entries in (table, bag) order with the width of the
 * indices (index_bits). d_indice_weights NULL = unweighted. d_output is
 * [B, total_D] of output_ty, row-major; columns of table t start at
 * D_offsets[t]. The first forward with a new B uploads a per-wave work list
 * (allocates); later ones reuse it.
 * output_ty FBGEMM_AMD_INT8 is the reference GPU operator's quantized pooled
 * output (embedding_forward_quantized_split_nbit_kernel_template.cu:535-566;
 * shape: fbgemm_gpu/fbgemm_gpu/sparse_ops.py:571-577): d_output is uint8
 * [B, total_D + 8 T]; per bag and table, the pooled fp32 vector quantized
 * row-wise to 8 bits as FloatToFused8BitRowwiseQuantized does (D_t bytes, fp32
 * scale, fp32 bias), table t starting at byte D_offsets[t] + 8 t. Tables of
 * the regular shapes are quantized in the lookup kernel's own output stage, as
 * in the reference; tables of other shapes (and forwards that cut their bags
 * into segments) go as floats through a plan-owned fp32 [B, total_D] scratch
 * and one more launch. */
int fbgemm_amd_tbe_forward(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t pooling_mode,
    const float* d_indice_weights, int32_t output_ty, void* d_output,
    void* d_status, void* stream);

/* The same forward with the pruned-row remap fused in: d_indices hold LOGICAL
 * ids; for a table with a mapping (index_remappings_offsets[t+1] >
 * index_remappings_offsets[t], both as in pruned_array_lookup) the physical
 * row is index_remappings[offsets[t] + id], -1 = pruned = skipped; tables
 * without a mapping take their ids as they are. Equal, bit for bit, to
 * fbgemm_amd_pruned_array_lookup followed by fbgemm_amd_tbe_forward (the order
 * of split_table_batched_embeddings_ops_inference.py:1067-1152) without the
 * round trip of the dense indices through HBM. A logical id outside its
 * mapping is reported as out of range. index_remappings_offsets_numel must be
 * T + 1 with T the plan's tables (the operator's features). No counterpart as
 * one call in the reference. */
int fbgemm_amd_tbe_forward_pruned(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t pooling_mode,
    const float* d_indice_weights, int32_t output_ty, void* d_output,
    const void* d_index_remappings, int32_t remap_bits,
    const int64_t* d_index_remappings_offsets, int64_t index_remappings_offsets_numel,
    void* d_status, void* stream);

/* A compact form of the mappings for the call above. No counterpart in the
 * reference. For every table whose mapping is order-preserving (its kept rows
 * are numbered 0, 1, 2, ... in logical order: what embedding_bag_rowwise_prune
 * and the inference converter produce) the plan builds, on the device, 2 bits per
 * logical row (a kept-row bitmap with a running count per 32 rows) and the
 * forwards compute the physical row from that instead of fetching a 4- or 8-byte
 * entry of a table-sized array: the same integers, from a structure that fits
 * the caches. Tables whose mapping is anything else keep reading the array.
 * d_index_remappings / remap_bits as in the forward; index_remappings_offsets is
 * the HOST copy of the T+1 offsets. The forwards use the records whenever they
 * are passed the same d_index_remappings pointer, and then bound and slice the
 * mappings with the offsets given HERE (the plan keeps a device copy), whatever
 * offsets the forward is handed; call this again after the array's contents or
 * its offsets change (NULL array = drop the records). Allocates; synchronizes
 * `stream`. fbgemm_amd_tbe_plan_rank_tables returns how many tables use records. */
int fbgemm_amd_tbe_plan_set_index_remappings(
    fbgemm_amd_tbe_plan* plan, const void* d_index_remappings, int32_t remap_bits,
    const int64_t* index_remappings_offsets, int64_t index_remappings_offsets_numel, void* stream);
int32_t fbgemm_amd_tbe_plan_rank_tables(const fbgemm_amd_tbe_plan* plan);

/* Select FBGEMM_AMD_ACC_EXACT (the default of a new plan) or FBGEMM_AMD_ACC_FAST
 * for the forwards of a plan. No counterpart in the reference. */
int fbgemm_amd_tbe_plan_set_accumulate(fbgemm_amd_tbe_plan* plan, int32_t mode);

/* A plan caches, per (batch size, stream), the work lists of its forwards and the
 * scratch of the bag scheduler; past 16 entries the least recently used one that
 * no forward under stream capture has touched is dropped. This call drops ALL of
 * them (after a device synchronize), including those a captured graph may hold:
 * graphs that contain forwards of this plan must be captured again afterwards.
 * fbgemm_amd_tbe_plan_cached_work returns the number of cached entries. No
 * counterpart in the reference. */
int fbgemm_amd_tbe_plan_trim(fbgemm_amd_tbe_plan* plan);
int64_t fbgemm_amd_tbe_plan_cached_work(const fbgemm_amd_tbe_plan* plan);
/* How many of the cached entries a forward under stream capture has touched (a
 * graph may hold their addresses): a cache of plans must not destroy a plan
 * while this is not 0 unless its owner knows the graphs are gone. */
int64_t fbgemm_amd_tbe_plan_pinned_work(fbgemm_amd_tbe_plan* plan);

/* Tables of FBGEMM_AMD_FP8 rows (D bytes per row, no scale/bias) are decoded
 * with the operator's fp8_exponent_bits / fp8_exponent_bias
 * (Float8ToFloat_ref, src/RefImplementations.cc:184-214; the pooled arithmetic
 * is EmbeddingSpMDMFP8_ref's, :1544-1616: acc = fma(w, value, acc)). Set them
 * before the first forward of a plan that holds such tables; an index of -1 is
 * skipped as for every other row type. */
int fbgemm_amd_tbe_plan_set_fp8(fbgemm_amd_tbe_plan* plan, int32_t exponent_bits, int32_t exponent_bias);

/* The forward without pooling (PoolingMode.NONE, "sequence" output;
 * embedding_forward_quantized_host_cpu.cpp:113-139 and
 * embedding_forward_quantized_cpu_template.cpp:283-296,390-420): d_output is
 * [indices_numel, D] of output_ty, row i the row d_indices[i] of the table
 * whose slice of d_offsets holds position i, converted like a bag of one
 * (unweighted); an index of -1 gives a row of zeros. All tables share D (the
 * operator passes the largest of its max_*_D). output_ty FBGEMM_AMD_INT8 /
 * FBGEMM_AMD_INT4 copies the stored row (fp16 scale, fp16 bias, elements:
 * D + 4 bytes, resp. (D + 8) / 2 bytes per output row) and needs every table
 * to be of that type (src/RefImplementations.cc:1235-1253,1466-1484). */
int fbgemm_amd_tbe_forward_nobag(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t D, int32_t output_ty,
    void* d_output, void* d_status, void* stream);

/* Rows the plan inferred for table t (what an index is checked against). */
int64_t fbgemm_amd_tbe_plan_num_rows(const fbgemm_amd_tbe_plan* plan, int32_t t);
/* Padded row bytes of table t. */
int64_t fbgemm_amd_tbe_plan_row_bytes(const fbgemm_amd_tbe_plan* plan, int32_t t);

/* ---- pruned-row remap ------------------------------------------------------ *
 * Replaces pruned_array_lookup
 * (embedding_forward_quantized_cpu_template.cpp:605-659,
 * embedding_forward_quantized_split_lookup.cu:120-168): position-preserving,
 * d_dense[i] = remap[remap_offsets[t] + indices[i]] for tables that own a
 * mapping (remap_offsets[t+1] > remap_offsets[t]), a copy otherwise. An id
 * outside its table's mapping yields -1 (the reference reads out of bounds). */
int fbgemm_amd_pruned_array_lookup(
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t offsets_numel, const void* d_index_remappings, int32_t remap_bits,
    const int64_t* d_index_remappings_offsets, int32_t T, void* d_dense,
    void* stream);

/* ---- in-place row update of a table-batched weights buffer ----------------- *
 * Replaces emb_inplace_update
 * (fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update.cu:28-101,207-282,
 * CPU form embedding_inplace_update_cpu.cpp:25-70; schema :257-258; caller
 * embedding_inplace_update_internal,
 * fbgemm_gpu/fbgemm_gpu/split_table_batched_embeddings_ops_inference.py:2057-2144):
 * for update i the padded row d_update_row_idx[i] of table d_update_table_idx[i]
 * (fbgemm_amd_tbe_plan_row_bytes bytes) is overwritten with the bytes at
 * d_update_weights + d_update_offsets[i]. Tables, row sizes, placements and row
 * counts come from the plan. Beyond the reference, which checks nothing: a row id
 * of -1 (a pruned row, see below) is skipped; a table outside [0, T), another row
 * outside its table, or an update that would read past update_weights_bytes is
 * skipped and recorded in d_status (out-of-range / overrun bits; may be NULL:
 * then it is only skipped). Two updates of one row in a call race, as in the
 * reference's kernel. Asynchronous; forwards that should see the rows must be
 * ordered after it on `stream`. */
int fbgemm_amd_tbe_inplace_update(
    fbgemm_amd_tbe_plan* plan, void* d_dev_weights, void* d_uvm_weights,
    const void* d_update_weights, int64_t update_weights_bytes,
    const int32_t* d_update_table_idx, const void* d_update_row_idx, int32_t row_index_bits,
    const int64_t* d_update_offsets, int64_t n, void* d_status, void* stream);

/* Replaces pruned_array_lookup_from_row_idx (embedding_inplace_update.cu:359-465,
 * embedding_inplace_update_cpu.cpp:199-251): the logical rows of an update become
 * physical rows, d_dense[i] = index_remappings[offsets[t_i] + row_i] where table
 * t_i owns a mapping and row_i otherwise. A row outside its mapping or a table
 * outside [0, T) yields -1 (the reference reads out of bounds). */
int fbgemm_amd_pruned_array_lookup_from_row_idx(
    const void* d_update_row_idx, int32_t index_bits, const int32_t* d_update_table_idx, int64_t n,
    const void* d_index_remappings, int32_t remap_bits, const int64_t* d_index_remappings_offsets,
    int32_t T, void* d_dense, void* stream);

/* ---- index operators that run before the lookup ---------------------------- *
 *
 * bounds_check_indices (fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:76-219,
 * schema :240-256; the step before the lookup in
 * split_table_batched_embeddings_ops_inference.py:1067-1124). In place on
 * d_indices / d_offsets (same width). bounds_check_mode: 0 FATAL, 1 WARNING,
 * 2 IGNORE (embedding_common.h:44-48).
 *   WARNING / IGNORE: offsets[last] becomes indices_numel; every offset is
 *     clamped to [0, indices_numel] and raised to the largest offset before it
 *     (what the reference's sequential loop leaves); an index other than -1
 *     outside [0, rows_per_table[t]) becomes 0. WARNING zeroes d_warning[0]
 *     first and counts one per repaired last offset, per bad bag and per bad
 *     index, like the reference's counter.
 *   FATAL: nothing is modified; the conditions the reference raises on are
 *     ORed into d_status (FBGEMM_AMD_ERR_LENGTH_MISMATCH: last offset !=
 *     indices_numel; FBGEMM_AMD_ERR_BAG_OVERRUN: offsets negative, decreasing
 *     or beyond indices_numel; FBGEMM_AMD_ERR_INDEX_OUT_OF_RANGE, with the
 *     first offending position). The reference's GPU kernel asserts on the
 *     device instead, which takes the process down.
 * d_B_offsets: NULL, or int32[T+1] first bag of every table (variable batch
 * sizes). Uses library-owned scratch: calls must be ordered on one stream. */
int fbgemm_amd_bounds_check_indices(
    const int64_t* d_rows_per_table, int32_t T, void* d_indices, void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t bounds_check_mode, int64_t* d_warning,
    const int32_t* d_B_offsets, void* d_status, void* stream);

/* pruned_hashmap_lookup (embedding_forward_quantized_cpu_template.cpp:524-603; GPU
 * embedding_forward_quantized_split_lookup.cu:19-118): d_hash_table holds
 * [slots][2] (sparse id, dense id) pairs of hash_bits each, -1 = empty, built by
 * the reference's pruned_hashmap_insert (linear probing from MurmurHash3's
 * finalizer of the id, 32- or 64-bit after the index width, modulo the table's
 * capacity). d_dense[i] = the dense id of d_indices[i], -1 when absent, a copy
 * for tables with an empty slot range. */
int fbgemm_amd_pruned_hashmap_lookup(
    const void* d_indices, const void* d_offsets, int32_t index_bits, int64_t offsets_numel,
    const void* d_hash_table, int32_t hash_bits, const int64_t* d_hash_table_offsets, int32_t T,
    void* d_dense, void* stream);

/* pruned_hashmap_insert (embedding_forward_quantized_cpu_template.cpp:124-201;
 * the reference has this operator on the CPU only and its GPU module calls
 * it there, split_table_batched_embeddings_ops_inference.py:2001-2010): HOST
 * pointers, runs on the calling thread. Inserts (indices[i], dense_indices[i])
 * of every table's slice into that table's slots of h_hash_table ([slots][2],
 * -1 = empty), skipping pairs whose dense id is -1, by linear probing from the
 * same hash as the lookup. Returns FBGEMM_AMD_E_ARG when a table has no empty
 * slot left (the reference would not return). */
int fbgemm_amd_pruned_hashmap_insert_host(
    const void* h_indices, const void* h_dense_indices, const void* h_offsets, int32_t index_bits,
    int64_t offsets_numel, void* h_hash_table, int32_t hash_bits, const int64_t* h_hash_table_offsets, int32_t T);

/* ---- row-wise quantizers: producers and readers of the row formats ---------- *
 *
 * fp32 / fp16 rows [rows][cols] -> fused quantized rows, bit for bit what the
 * reference's CPU routines write:
 *   bit_rate 2 / 4 / 8, sb_float 0: FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf
 *     (src/QuantUtils.cc:534-611): packed elements, then fp16 scale, fp16 bias;
 *   bit_rate 8, sb_float 1: FloatOrHalfToFused8BitRowwiseQuantizedSBFloat
 *     (src/QuantUtils.cc:677-718): bytes, then fp32 scale, fp32 bias.
 * layout FBGEMM_AMD_QLAYOUT_TRAILER keeps that order; FBGEMM_AMD_QLAYOUT_TBE
 * writes the table-batched operator's rows, fp16 scale and bias FIRST, then
 * the elements, as quantize_embs rearranges them
 * (fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:47-70; with sb_float 1 the fp32
 * pair is rounded to fp16, as there). out_row_stride is in bytes (>= the row's
 * size: padding bytes are left alone). */
enum { FBGEMM_AMD_QLAYOUT_TRAILER = 0, FBGEMM_AMD_QLAYOUT_TBE = 1 };
int fbgemm_amd_quantize_rowwise(
    const void* d_input, int32_t input_ty, int64_t rows, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int64_t out_row_stride, void* d_output, void* stream);

/* The same with extremes the caller brings: the `rowwise_min_max` argument of
 * FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf / FloatOrHalfToFused8BitRowwiseQuantizedSBFloat
 * (include/fbgemm/QuantUtils.h:277-283, :311-317; src/QuantUtilsAvx2.cc:1605-1628, :1831-1853).
 * d_rowwise_min_max holds [rows][2] values of the input's type, minimum then
 * maximum, which take the place of the row's own extremes; null means "find
 * them", as the call above. Elements outside the extremes given: the 2 / 4 / 8
 * bit fp16-pair formats saturate to 0 .. 2^bit_rate - 1; the 8-bit fp32-pair
 * format does what the reference's vector code does, saturate in the leading
 * whole groups of 32 columns and keep the low byte of the rounded integer in
 * the columns behind them. */
int fbgemm_amd_quantize_rowwise_min_max(
    const void* d_input, int32_t input_ty, int64_t rows, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int64_t out_row_stride, void* d_output, const void* d_rowwise_min_max, void* stream);

/* The inverses (src/QuantUtils.cc:743-789 FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf,
 * :847-892 Fused8BitRowwiseQuantizedSBFloatToFloatOrHalf): element =
 * float(double(scale) * q + double(bias)), written as fp32, fp16 (round to
 * nearest even) or bf16 ((bits + 0x8000) >> 16); output [rows][cols], dense. */
int fbgemm_amd_dequantize_rowwise(
    const void* d_input, int64_t rows, int64_t in_row_stride, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int32_t output_ty, void* d_output, void* stream);

/* fp32 <-> 8-bit float (hfp8) element-wise, `n` elements: the operators
 * FloatToHFP8Quantized / HFP8QuantizedToFloat
 * (fbgemm_gpu/src/quantize_ops/quantize_ops_cpu.cpp:531-620,
 * fbgemm_gpu/include/fbgemm_gpu/quantize_ops_utils.h:29-110; the same arithmetic as
 * FloatToFloat8_ref / Float8ToFloat_ref, src/RefImplementations.cc:126-214), which
 * produce and read back the rows of FP8 tables (quantize_embs,
 * fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:36-45). |x| is clamped to max_pos,
 * rounding is to nearest even, values below the smallest normal keep gradual
 * underflow. */
int fbgemm_amd_float_to_hfp8(const float* d_input, int64_t n, int32_t ebits, int32_t exponent_bias, float max_pos,
                             uint8_t* d_output, void* stream);
int fbgemm_amd_hfp8_to_float(const uint8_t* d_input, int64_t n, int32_t ebits, int32_t exponent_bias, float* d_output,
                             void* stream);

/* fbgemm::compressed_indices_remap (include/fbgemm/FbgemmEmbedding.h:392-401,
 * src/RefImplementations.cc:2308-2333): the core library's pruned-row remap, which
 * compacts. Entries whose row is pruned (d_mapping[index] == -1) are dropped, the
 * others become their physical row and move up, per-sample weights (optional) move
 * with them; d_out_offsets[i] = entries that stay before bag i, d_out_offsets[0] =
 * offsets[0]. Indices and offsets share index_bits; offsets must not decrease (the
 * reference then walks positions offsets[0] .. offsets[last]-1 in order). Beyond the
 * reference: mapping_numel bounds the indices (an index outside the mapping is dropped
 * and recorded in d_status instead of being read; d_status may be NULL: then it is
 * only dropped). Outputs must not alias inputs.
 * Reads offsets[0] and offsets[last] back first (synchronizes `stream`), then runs
 * asynchronously; uses library-owned scratch (calls must be ordered on one stream). */
int fbgemm_amd_compressed_indices_remap(
    int32_t offsets_numel, const void* d_indices, int32_t index_bits, const int32_t* d_mapping, int64_t mapping_numel,
    const void* d_offsets, const float* d_weights, void* d_out_indices, void* d_out_offsets, float* d_out_weights,
    void* d_status, void* stream);

/* embedding_bag_rowwise_prune (fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2836-2893,
 * which ends in at::native::_rowwise_prune; the converter's pruning step,
 * fbgemm_gpu/fbgemm_gpu/split_embedding_inference_converter.py:75-93), in two calls
 * because the size of the result depends on the data.
 * _map: row i stays when indicator[i] (|indicator[i]| with use_abs) > threshold, or
 * when the rows kept so far plus all rows still to come do not exceed
 * min_non_pruned_rows; d_remap[rows] (int32 or int64) receives the new row id or -1,
 * *num_kept (host) the number of rows that stay. Synchronizes `stream`.
 * _gather: d_output[remap[i]] = d_weights[i] for the rows that stay; rows of
 * row_bytes bytes, output_rows = the num_kept the map gave. */
int fbgemm_amd_rowwise_prune_map(const float* d_indicator, int64_t rows, double threshold, int32_t use_abs,
                                 int64_t min_non_pruned_rows, int32_t index_bits, void* d_remap, int64_t* num_kept,
                                 void* stream);
int fbgemm_amd_rowwise_prune_gather(const void* d_weights, int64_t rows, int64_t row_bytes, const void* d_remap,
                                    int32_t index_bits, void* d_output, int64_t output_rows, void* stream);

/* Wait for everything enqueued on `stream` (hipStreamSynchronize), for callers
 * of the asynchronous entry points that hold no HIP headers. */
int fbgemm_amd_stream_synchronize(void* stream);

/* ---- row-size arithmetic (host, no GPU) ------------------------------------ *
 * embedding_common.h:189-225. */
int32_t fbgemm_amd_unpadded_row_size_in_bytes(int32_t dim, int32_t weight_ty, int32_t scale_bias_bytes);
int32_t fbgemm_amd_padded_row_size_in_bytes(int32_t dim, int32_t weight_ty, int32_t row_alignment, int32_t scale_bias_bytes);

#ifdef __cplusplus
}
#endif
#endif /* FBGEMM_AMD_H_ */
