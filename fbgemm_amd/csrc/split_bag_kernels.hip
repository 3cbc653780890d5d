// Few, long bags: a bag is cut into K segments that are pooled as bags of their
// own (by the ordinary lookup kernels, into fp32 partial sums) and added up
// afterwards in segment order. A launch of ten bags of a hundred rows, the shape
// of the reference's own microbenchmark (bench/EmbeddingSpMDMNBitBenchmark.cc:47-63),
// otherwise runs on a handful of waves as a chain of dependent memory round trips.
//
// The sum of the segments' partial sums is not the reference's sequence of
// roundings (it adds the rows of a bag one after the other into one accumulator),
// so this path belongs to the tolerance-grade accumulate mode only. The order of
// the additions is fixed (segment 0, 1, 2, ...): results do not change from run
// to run. No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "lookup_common.h"

namespace fbgemm_amd {

namespace {

__device__ __forceinline__ int64_t sb_read_offset(const void* p, int is64, int64_t i) {
  return is64 ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}

// voff[(t * B + b) * K + k] = where segment k of bag (t, b) starts in the index array
// (relative to offsets[0] when `relative`: single-table calls), and one entry more for the
// end of the last segment. Segments hold ceil(len / K) entries; the last ones may be empty.
__global__ __launch_bounds__(256) void split_offsets_kernel(const void* offsets, int off64, int64_t bags, int32_t K,
                                                            int relative, int64_t index_size, int64_t* voff, Status* status) {
  const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= bags) return;
  const int64_t base = relative ? sb_read_offset(offsets, off64, 0) : 0;
  const int64_t o0 = sb_read_offset(offsets, off64, v) - base;
  const int64_t o1 = sb_read_offset(offsets, off64, v + 1) - base;
  int64_t len = o1 - o0;
  if (len < 0) len = 0; // the lookup reports it: the last segment then ends before it starts
  const int64_t seg = (len + K - 1) / K;
  for (int k = 0; k < K; ++k) {
    const int64_t s = (int64_t)k * seg;
    voff[v * K + k] = o0 + (s < len ? s : len);
  }
  if (v == bags - 1) {
    voff[bags * K] = o1;
    if (relative && o1 != index_size) atomicOr(&status->bits, ERR_LENGTH_MISMATCH);
  }
}

__device__ __forceinline__ uint32_t sb_half_bits(float f) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f); }

// out[b][table t's columns] = (sum over k of partial[(b * K + k)][those columns]) * (1 / len when mean pooling),
// converted like the lookup's own output stage. One workgroup per (bag, table).
__global__ __launch_bounds__(256) void combine_segments_kernel(const float* partial, int64_t partial_stride, int32_t B, int32_t K,
                                                               const int32_t* D_offsets, int32_t single_D, const void* offsets,
                                                               int off64, int normalize, void* out, int32_t out_ty,
                                                               int64_t out_stride) {
  const int b = blockIdx.x, t = blockIdx.y;
  const int c0 = D_offsets ? D_offsets[t] : 0;
  const int c1 = D_offsets ? D_offsets[t + 1] : single_D;
  float inv_len = 1.0f;
  if (normalize) {
    const int64_t v = (int64_t)t * B + b;
    const int64_t len = sb_read_offset(offsets, off64, v + 1) - sb_read_offset(offsets, off64, v);
    if (len > 0 && len <= 0x7fffffffLL) inv_len = 1.0f / (float)(int)len;
  }
  const float* p = partial + ((int64_t)b * K) * partial_stride;
  for (int c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
    float sum = p[c];
    for (int k = 1; k < K; ++k) sum += p[(int64_t)k * partial_stride + c];
    if (normalize) sum *= inv_len;
    const int64_t o = (int64_t)b * out_stride + c;
    if (out_ty == ST_FP32) reinterpret_cast<float*>(out)[o] = sum;
    else if (out_ty == ST_FP16) reinterpret_cast<uint16_t*>(out)[o] = (uint16_t)sb_half_bits(sum);
    else reinterpret_cast<uint16_t*>(out)[o] = (uint16_t)((__builtin_bit_cast(uint32_t, sum) + 0x8000u) >> 16);
  }
}

} // namespace

hipError_t launch_split_offsets(const void* offsets, bool off64, int64_t bags, int32_t K, bool relative, int64_t index_size,
                                int64_t* voff, Status* status, hipStream_t stream) {
  if (bags <= 0) return hipSuccess;
  hipLaunchKernelGGL(split_offsets_kernel, dim3((unsigned)((bags + 255) / 256)), dim3(256), 0, stream, offsets, off64 ? 1 : 0,
                     bags, K, relative ? 1 : 0, index_size, voff, status);
  return hipGetLastError();
}

hipError_t launch_combine_segments(const float* partial, int64_t partial_stride, int32_t B, int32_t K, int32_t T,
                                   const int32_t* D_offsets, int32_t single_D, const void* offsets, bool off64, bool normalize,
                                   void* out, int32_t out_ty, int64_t out_stride, hipStream_t stream) {
  if (B <= 0 || T <= 0) return hipSuccess;
  hipLaunchKernelGGL(combine_segments_kernel, dim3((unsigned)B, (unsigned)T), dim3(256), 0, stream, partial, partial_stride, B, K,
                     D_offsets, single_D, offsets, off64 ? 1 : 0, normalize ? 1 : 0, out, out_ty, out_stride);
  return hipGetLastError();
}

} // namespace fbgemm_amd
