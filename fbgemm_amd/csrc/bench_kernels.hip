// Yardsticks for benchmarks and profiles, built into a library of their own
// (libfbgemm_amd_bench.so, declared in include/fbgemm_amd_bench.h): nothing here
// is on the product path and nothing has a counterpart in the reference.
//  * a plain copy of known size, against which the hardware byte counters of the
//    lookup kernels are scaled;
//  * a streaming read;
//  * gathers of random rows with 16-byte lanes, in the access shapes of the
//    lookup kernels (rows in flight per lane group, 4-byte aligned loads), with
//    plain loads into registers or with gfx950's 16-byte loads straight into LDS.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fbgemm_amd_bench.h"

namespace {

struct __attribute__((packed, aligned(4))) Dwordx4 { uint32_t v[4]; };

__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4* src, uint4* dst, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// Every lane reads 16 bytes per load, 8 loads in flight, consecutive lanes
// consecutive addresses. One dword per wave is written so that the loads stay.
constexpr int STREAM_BLOCKS = 256 * 8, STREAM_THREADS = 256;
__global__ __launch_bounds__(STREAM_THREADS) void stream_read_kernel(const uint4* src, int64_t n16, uint32_t* sink) {
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
// `stride` bytes apart, DEPTH rows per lane group in flight. byte_offset = 4
// gives the 4-byte-aligned loads of rows whose data follows a 4-byte header.
// Row ids are clamped to the table.
template <int DEPTH>
__global__ __launch_bounds__(64) void gather_lines_kernel(const uint8_t* table, int64_t rows, int64_t stride, int32_t lanes,
                                                          int32_t byte_offset, const int32_t* idx, int64_t n, uint32_t* sink) {
  const int lane = threadIdx.x;
  const int groups = 64 / lanes;
  const int grp = lane / lanes, sub = lane - grp * lanes;
  const int64_t per_wave = (int64_t)groups * DEPTH;
  uint32_t acc = 0;
  for (int64_t base = (int64_t)blockIdx.x * per_wave; base < n; base += (int64_t)gridDim.x * per_wave) {
    Dwordx4 v[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const int64_t i = base + (int64_t)grp * DEPTH + k;
      int64_t row = (i < n && grp < groups) ? (int64_t)idx[i] : 0;
      row = row < 0 ? 0 : (row >= rows ? rows - 1 : row);
      v[k] = *reinterpret_cast<const Dwordx4*>(table + row * stride + byte_offset + sub * 16);
    }
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) acc ^= v[k].v[0] ^ v[k].v[1] ^ v[k].v[2] ^ v[k].v[3];
  }
  if (lane == 0) sink[blockIdx.x] = acc;
}

// The same gather with the 16-byte loads that write LDS directly (no registers
// for the data in flight): lane l of load k lands in buf[k][l]. 16-byte aligned
// addresses only (byte_offset a multiple of 16, stride a multiple of 16).
typedef const void __attribute__((address_space(1)))* global_ptr;
typedef void __attribute__((address_space(3)))* lds_ptr;
__global__ __launch_bounds__(64) void gather_lines_lds_kernel(const uint8_t* table, int64_t rows, int64_t stride, int32_t lanes,
                                                              int32_t byte_offset, const int32_t* idx, int64_t n, uint32_t* sink) {
  constexpr int DEPTH = 8;
  __shared__ __attribute__((aligned(16))) uint4 buf[DEPTH][64];
  const int lane = threadIdx.x;
  const int groups = 64 / lanes;
  const int grp = lane / lanes, sub = lane - grp * lanes;
  const int64_t per_wave = (int64_t)groups * DEPTH;
  uint32_t acc = 0;
  for (int64_t base = (int64_t)blockIdx.x * per_wave; base < n; base += (int64_t)gridDim.x * per_wave) {
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const int64_t i = base + (int64_t)grp * DEPTH + k;
      int64_t row = (i < n && grp < groups) ? (int64_t)idx[i] : 0;
      row = row < 0 ? 0 : (row >= rows ? rows - 1 : row);
      __builtin_amdgcn_global_load_lds((global_ptr)(table + row * stride + byte_offset + sub * 16), (lds_ptr)&buf[k][0], 16, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): every load has written LDS
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const uint4 v = buf[k][lane];
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) sink[blockIdx.x] = acc;
}

thread_local char g_err[256] = "";
int fail(const char* msg) {
  snprintf(g_err, sizeof(g_err), "%s", msg);
  return -1;
}
int hip_fail(hipError_t e) {
  snprintf(g_err, sizeof(g_err), "%s", hipGetErrorString(e));
  return -2;
}

} // namespace

extern "C" {

const char* fbgemm_amd_bench_last_error(void) { return g_err; }

int fbgemm_amd_bench_calibration_copy(const void* d_src, void* d_dst, int64_t bytes, void* stream) {
  if (bytes < 0 || bytes % 16 || (bytes && (!d_src || !d_dst))) return fail("bad calibration copy arguments");
  if (bytes == 0) return 0;
  hipLaunchKernelGGL(calibration_copy_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const uint4*)d_src, (uint4*)d_dst, bytes / 16);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e);
}

int fbgemm_amd_bench_stream_read(const void* d_src, int64_t bytes, void* d_sink, int64_t sink_dwords, void* stream) {
  if (!d_src || !d_sink || bytes < 16) return fail("bad stream read arguments");
  if (sink_dwords < (int64_t)STREAM_BLOCKS * STREAM_THREADS / 64) return fail("the sink of the streaming read needs 8192 dwords");
  hipLaunchKernelGGL(stream_read_kernel, dim3(STREAM_BLOCKS), dim3(STREAM_THREADS), 0, (hipStream_t)stream, (const uint4*)d_src, bytes / 16,
                     (uint32_t*)d_sink);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e);
}

int fbgemm_amd_bench_gather(const void* d_table, int64_t rows, int64_t row_stride, int32_t lanes_per_row, int32_t byte_offset,
                            const int32_t* d_rows, int64_t n, void* d_sink, int64_t sink_dwords, int32_t waves, int32_t mode,
                            void* stream) {
  if (!d_table || !d_rows || !d_sink || n <= 0 || rows <= 0) return fail("bad gather arguments");
  if (lanes_per_row < 1 || lanes_per_row > 64) return fail("lanes_per_row must be 1..64");
  if (waves < 1 || (int64_t)waves > sink_dwords) return fail("the sink holds fewer dwords than there are waves");
  if (row_stride < (int64_t)byte_offset + 16 * (int64_t)lanes_per_row || byte_offset < 0 || byte_offset % 4 || row_stride % 4)
    return fail("the bytes a row's lanes read do not fit its stride, or are not 4-byte aligned");
  const dim3 grid((unsigned)waves), block(64);
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* t = (const uint8_t*)d_table;
  uint32_t* sink = (uint32_t*)d_sink;
  if (mode == FBGEMM_AMD_BENCH_GATHER_REGISTERS)
    hipLaunchKernelGGL(gather_lines_kernel<8>, grid, block, 0, s, t, rows, row_stride, lanes_per_row, byte_offset, d_rows, n, sink);
  else if (mode == FBGEMM_AMD_BENCH_GATHER_REGISTERS_16)
    hipLaunchKernelGGL(gather_lines_kernel<16>, grid, block, 0, s, t, rows, row_stride, lanes_per_row, byte_offset, d_rows, n, sink);
  else if (mode == FBGEMM_AMD_BENCH_GATHER_LDS) {
    if (byte_offset % 16 || row_stride % 16 || (uintptr_t)d_table % 16) return fail("loads into LDS need 16-byte aligned addresses");
    hipLaunchKernelGGL(gather_lines_lds_kernel, grid, block, 0, s, t, rows, row_stride, lanes_per_row, byte_offset, d_rows, n, sink);
  } else {
    return fail("unknown gather mode");
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e);
}

} // extern "C"
