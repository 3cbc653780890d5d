// Yardsticks for the two access patterns a pooled lookup is made of, so that its
// achieved rate can be held against what this GPU sustains for the pattern
// itself: a streaming read, and a gather of random rows with 16-byte lanes
// (rows in flight per lane as in the lookup kernels). No counterpart in the
// reference; nothing here is on the product path.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fbgemm_amd {

struct __attribute__((packed, aligned(4))) CeilDwordx4 { uint32_t v[4]; };

// Every lane reads 16 bytes per load, 8 loads in flight, consecutive lanes
// consecutive addresses. One dword per wave is written so that the loads stay.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* src, int64_t n16, uint32_t* sink) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = src[i + k * stride];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
  }
  for (; i < n16; i += stride) {
    const uint4 v = src[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if ((threadIdx.x & 63) == 0) sink[((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6] = acc;
}

// `lanes` consecutive lanes read 16 bytes each of row idx[.]: bytes
// [byte_offset + 16 k, byte_offset + 16 k + 16) of the row for lane k, rows
// `stride` bytes apart. A wave has 8 rows per lane group in flight, as the
// lookup kernels do. byte_offset = 4 gives the 4-byte-aligned loads of rows whose
// data follows a 4-byte header.
__global__ __launch_bounds__(64) void gather_lines_kernel(const uint8_t* table, int64_t stride, int32_t lanes, int32_t byte_offset,
                                                          const int32_t* idx, int64_t n, uint32_t* sink) {
  const int lane = threadIdx.x;
  const int groups = 64 / lanes;
  const int grp = lane / lanes, sub = lane - grp * lanes;
  const int64_t per_wave = (int64_t)groups * 8;
  uint32_t acc = 0;
  for (int64_t base = (int64_t)blockIdx.x * per_wave; base < n; base += (int64_t)gridDim.x * per_wave) {
    CeilDwordx4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t i = base + (int64_t)grp * 8 + k;
      const int64_t row = i < n ? (int64_t)idx[i] : 0;
      v[k] = *reinterpret_cast<const CeilDwordx4*>(table + row * stride + byte_offset + sub * 16);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) acc ^= v[k].v[0] ^ v[k].v[1] ^ v[k].v[2] ^ v[k].v[3];
  }
  if (lane == 0) sink[blockIdx.x] = acc;
}

hipError_t launch_stream_read(const void* src, int64_t bytes, uint32_t* sink, hipStream_t stream) {
  const int64_t n16 = bytes / 16;
  if (n16 <= 0) return hipSuccess;
  hipLaunchKernelGGL(stream_read_kernel, dim3(256 * 8), dim3(256), 0, stream, (const uint4*)src, n16, sink);
  return hipGetLastError();
}

hipError_t launch_gather_lines(const void* table, int64_t stride, int32_t lanes, int32_t byte_offset, const int32_t* idx,
                               int64_t n, uint32_t* sink, int32_t waves, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(gather_lines_kernel, dim3((unsigned)waves), dim3(64), 0, stream, (const uint8_t*)table, stride, lanes,
                     byte_offset, idx, n, sink);
  return hipGetLastError();
}

} // namespace fbgemm_amd
