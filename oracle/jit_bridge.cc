// TEST / BASELINE INFRASTRUCTURE ONLY.
//
// C bridge to the reference's production CPU kernels: the AVX2 / AVX-512 code
// that fbgemm::GenerateEmbeddingSpMDM*WithStrides generates at run time
// (include/fbgemm/FbgemmEmbedding.h:94-174, src/EmbeddingSpMDM.cc:972-1349,
// src/EmbeddingSpMDMNBit.cc:975-1258). The reference tree cannot build that
// path here (its asmjit submodule is empty), but PyTorch ships the same
// library inside libtorch_cpu.so and exports these factories, so this file
// includes PyTorch's copy of the header and links against it. It is used
// (a) as the timed CPU baseline of bench.py and (b) as a third opinion next
// to the C oracle and the reference's scalar code in the tests.
#include <fbgemm/FbgemmEmbedding.h>
#include <omp.h>

#include <cstdint>
#include <cstring>

namespace {

enum { ST_FP32 = 0, ST_FP16 = 1, ST_INT8 = 2, ST_INT4 = 3, ST_INT2 = 4, ST_BF16 = 5 };

template <typename Out>
bool run_one(int in_ty, int64_t D, int64_t output_size, int64_t index_size, int64_t data_size,
             const void* input, const int64_t* indices, const int64_t* offsets, const float* weights,
             bool normalize, Out* out, bool bf16_out, int64_t output_stride, int64_t input_stride,
             bool scale_bias_last) {
  const bool has_weight = weights != nullptr;
  switch (in_ty) {
    case ST_INT8: {
      auto k = fbgemm::GenerateEmbeddingSpMDMWithStrides<uint8_t, int64_t, int64_t, Out, true>(
          D, has_weight, normalize, 16, false, true, output_stride, input_stride, scale_bias_last, false,
          bf16_out, false);
      return k(output_size, index_size, data_size, static_cast<const uint8_t*>(input), indices, offsets, weights, out);
    }
    case ST_INT4:
    case ST_INT2: {
      auto k = fbgemm::GenerateEmbeddingSpMDMNBitWithStrides<int64_t, int64_t, Out, true>(
          in_ty == ST_INT4 ? 4 : 2, D, has_weight, normalize, 16, false, true, output_stride, input_stride,
          scale_bias_last, bf16_out, false, -1);
      return k(output_size, index_size, data_size, static_cast<const uint8_t*>(input), indices, offsets, weights, out);
    }
    case ST_FP16: {
      auto k = fbgemm::GenerateEmbeddingSpMDMWithStrides<uint16_t, int64_t, int64_t, Out, true>(
          D, has_weight, normalize, 16, false, true, output_stride, input_stride, scale_bias_last, false,
          bf16_out, false);
      return k(output_size, index_size, data_size, static_cast<const uint16_t*>(input), indices, offsets, weights, out);
    }
    case ST_FP32: {
      auto k = fbgemm::GenerateEmbeddingSpMDMWithStrides<float, int64_t, int64_t, Out, true>(
          D, has_weight, normalize, 16, false, true, output_stride, input_stride, scale_bias_last, false,
          bf16_out, false);
      return k(output_size, index_size, data_size, static_cast<const float*>(input), indices, offsets, weights, out);
    }
    default:
      return false;
  }
}

} // namespace

extern "C" {

// One pooled lookup with int64 indices and int64 offsets. Arguments as in
// oracle_embedding_spmdm (no remap). Returns 1 / 0 like the reference's bool.
int jit_embedding_spmdm(int in_ty, int64_t D, int64_t output_size, int64_t index_size, int64_t data_size,
                        const void* input, const int64_t* indices, const int64_t* offsets,
                        const float* weights, int normalize, void* out, int out_ty, int64_t output_stride,
                        int64_t input_stride, int scale_bias_last) {
  if (out_ty == ST_FP32)
    return run_one<float>(in_ty, D, output_size, index_size, data_size, input, indices, offsets, weights,
                          normalize != 0, static_cast<float*>(out), false, output_stride, input_stride,
                          scale_bias_last != 0);
  return run_one<uint16_t>(in_ty, D, output_size, index_size, data_size, input, indices, offsets, weights,
                           normalize != 0, static_cast<uint16_t*>(out), out_ty == ST_BF16, output_stride,
                           input_stride, scale_bias_last != 0);
}

// The table loop of the reference's CPU operator
// (fbgemm_gpu/codegen/inference/embedding_forward_quantized_cpu_template.cpp:343-515)
// over tables [t0, t1) of one problem: THREAD_LOCAL kernels, prefetch 16,
// offsets, scale/bias in front, output stride total_D. `threads` > 1 spreads
// the tables over OpenMP threads the way the operator does when
// FBGEMM_TBE_MAX_NUM_THREADS allows it. Returns 0, or 1 + the first failing table.
int jit_tbe_tables(int t0, int t1, const uint8_t* weights, const int64_t* weights_offsets,
                   const uint8_t* weights_tys, const int32_t* D_offsets, const int64_t* row_bytes,
                   const int64_t* num_rows, int64_t total_D, const int64_t* indices, const int64_t* offsets,
                   int64_t B, int pooling_mode, const float* indice_weights, int out_ty, void* output,
                   int threads) {
  int rc = 0;
  const size_t esz = out_ty == ST_FP32 ? 4 : 2;
#pragma omp parallel for schedule(dynamic) num_threads(threads > 0 ? threads : 1)
  for (int t = t0; t < t1; ++t) {
    const int ty = weights_tys[t];
    const int64_t D = D_offsets[t + 1] - D_offsets[t];
    const int64_t o0 = offsets[(int64_t)t * B], o1 = offsets[(int64_t)(t + 1) * B];
    const int64_t elem = ty == ST_FP32 ? 4 : (ty == ST_FP16 ? 2 : 1);
    const int ok = jit_embedding_spmdm(
        ty, D, B, o1 - o0, num_rows[t], weights + weights_offsets[t], indices + o0, offsets + (int64_t)t * B,
        indice_weights ? indice_weights + o0 : nullptr, pooling_mode == 1,
        static_cast<uint8_t*>(output) + (size_t)D_offsets[t] * esz, out_ty, total_D, row_bytes[t] / elem, 0);
    if (!ok) {
#pragma omp critical
      if (rc == 0 || 1 + t < rc) rc = 1 + t;
    }
  }
  return rc;
}

int jit_max_threads(void) { return omp_get_max_threads(); }

} // extern "C"
