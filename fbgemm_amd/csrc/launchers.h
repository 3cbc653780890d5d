// The kernel launchers the host side of the C ABI (c_api.cpp) calls, defined by the .hip files
// next to it. One list for both sides: the host-only build of c_api.cpp that runs under the
// address and undefined-behaviour sanitizers (tests/cpp/hip_stub) defines the same functions as
// stand-ins that launch nothing.
#pragma once
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {
hipError_t launch_lookup(const LookupArgs& a, bool idx64, hipStream_t stream);
hipError_t launch_lookup_lean(const LookupArgs& a, bool idx64, bool exact, bool wide4, hipStream_t stream);
hipError_t launch_lengths_to_offsets(const void* lengths, bool is64, int64_t n, int64_t* offsets, hipStream_t stream);
hipError_t launch_status_clear(Status* st, hipStream_t stream);
hipError_t launch_bag_order(const void* offsets, bool off64, int32_t B, int32_t T, BagEntry* order, hipStream_t stream);
hipError_t launch_sequence_lookup(const TableDesc* tables, const uint8_t* w0, const uint8_t* w1, const void* indices,
                                  bool idx64, const void* offsets, int32_t B, int32_t T, int64_t total_L, int32_t D,
                                  int32_t out_ty, void* out, int32_t fp8_shift, float fp8_mult, Status* status,
                                  hipStream_t stream);
hipError_t launch_row_lookup(const TableDesc& d, const uint8_t* table, const void* indices, bool idx64,
                             const float* weights, int64_t n, int32_t out_ty, void* out, int64_t out_stride_bytes,
                             int64_t copy_bytes, int32_t fp8_shift, float fp8_mult, Status* status, hipStream_t stream);
hipError_t launch_float_to_hfp8(const float* input, int64_t n, int32_t ebits, int32_t bias, float max_pos, uint8_t* output,
                                hipStream_t stream);
hipError_t launch_hfp8_to_float(const uint8_t* input, int64_t n, int32_t ebits, int32_t bias, float* output, hipStream_t stream);
hipError_t launch_inplace_update(const TableDesc* tables, int32_t T, uint8_t* w0, uint8_t* w1, const uint8_t* update,
                                 int64_t update_bytes, const int32_t* table_idx, const void* row_idx, bool idx64,
                                 const int64_t* update_offsets, int64_t n, int64_t max_row_bytes, Status* status,
                                 hipStream_t stream);
hipError_t launch_remap_row_idx(const void* rows, bool idx64, const int32_t* table_idx, const void* remap, bool remap64,
                                const int64_t* remap_offsets, int32_t T, int64_t n, void* dense, hipStream_t stream);
int64_t prune_partials(int64_t rows);
hipError_t launch_split_offsets(const void* offsets, bool off64, int64_t bags, int32_t K, bool relative, int64_t index_size,
                                int64_t* voff, Status* status, hipStream_t stream);
hipError_t launch_combine_segments(const float* partial, int64_t partial_stride, int32_t B, int32_t K, int32_t T,
                                   const int32_t* D_offsets, int32_t single_D, const void* offsets, bool off64, bool normalize,
                                   void* out, int32_t out_ty, int64_t out_stride, hipStream_t stream);
int64_t remap_rank_words(int64_t rows);
int64_t remap_rank_partials(int64_t rows);
hipError_t launch_remap_rank_build(const void* mapping, bool remap64, int64_t rows, RankRecord* records, int64_t* partial,
                                   int32_t* not_monotone, hipStream_t stream);
hipError_t launch_prune_map(const float* indicator, int64_t rows, double threshold, int use_abs, int64_t min_rows,
                            bool idx64, void* remap, int64_t* num_kept, int64_t* partial, hipStream_t stream);
hipError_t launch_prune_gather(const void* in, int64_t rows, int64_t row_bytes, const void* remap, bool idx64, void* out,
                               int64_t out_rows, hipStream_t stream);
hipError_t launch_compressed_indices_remap(const void* indices, bool idx64, const int32_t* mapping, int64_t mapping_numel,
                                           const void* offsets, int64_t offsets_numel, const float* weights, int64_t first,
                                           int64_t n, void* out_indices, void* out_offsets, float* out_weights,
                                           int64_t* before, int64_t* partial, int32_t* mapped, Status* status,
                                           hipStream_t stream);
hipError_t launch_quantize_segments(const float* input, int64_t lines, int32_t T, const int32_t* d_seg_offsets,
                                    int32_t total_D, int32_t max_D, uint8_t* output, const int32_t* d_tables,
                                    int32_t n_tables, hipStream_t stream);
hipError_t launch_bounds_check(const int64_t* rows_per_table, int32_t T, void* indices, void* offsets, bool is64,
                               int64_t num_indices, int64_t total_B, int64_t B, const int32_t* B_offsets, int mode,
                               int64_t* warning, int64_t* fixed, int64_t* partial, Status* status, hipStream_t stream);
int64_t bounds_check_partials(int64_t total_B);
hipError_t launch_quantize_rowwise(const void* input, bool half_in, int64_t rows, int32_t cols, int32_t bits,
                                   int32_t sb_float, int32_t layout, int64_t out_stride, void* output,
                                   const void* min_max, hipStream_t stream);
hipError_t launch_dequantize_rowwise(const void* input, int64_t rows, int64_t in_stride, int32_t cols, int32_t bits,
                                     int32_t sb_float, int32_t layout, int32_t output_ty, void* output,
                                     hipStream_t stream);
hipError_t launch_pruned_hashmap_lookup(const void* indices, const void* offsets, bool idx64, const void* hash_table,
                                        bool hash64, const int64_t* hash_table_offsets, int32_t B, int32_t T,
                                        void* dense, hipStream_t stream);
hipError_t launch_pruned_array_lookup(const void* indices, const void* offsets, bool idx64, const void* remap,
                                      bool remap64, const int64_t* remap_offsets, int32_t B, int32_t T,
                                      void* dense, hipStream_t stream);
} // namespace fbgemm_amd
