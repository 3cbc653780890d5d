// gfx950 kernels around the pooled lookup: the bag scheduler, lengths ->
// offsets, the status block, pruned_array_lookup, and
// the launchers the C ABI calls. The lookup kernels themselves are in
// lookup_general.h (any shape) and compiled one instance per translation unit.
#include "lookup_device.h"

namespace fbgemm_amd {

// ---- bag scheduler -------------------------------------------------------------
//
// One workgroup per window of SORT_WINDOW consecutive bags of a table orders them
// by length, longest first (counting sort over lengths, lengths >= SORT_BINS - 1
// share the first bin). Waves then take consecutive runs of the order, so the
// bags a wave pools side by side need the same number of rounds and no lane
// idles behind a long neighbour. Ties are placed in arrival order of the LDS
// atomics: the order may differ between runs, the results cannot (each bag is
// summed on its own). Windows for tables of many bags: a launch of many rounds of
// waves runs as fast over bags ordered inside windows of a few thousand as over
// tables ordered as a whole, and many workgroups order a table at once.
constexpr int SORT_BINS = 1024;
constexpr int SORT_WINDOW = 2048;
constexpr int SORT_WHOLE_TABLE = 8192;

__global__ __launch_bounds__(1024) void bag_order_kernel(const void* offsets, int off64, int32_t B_table, int32_t window,
                                                         BagEntry* order) {
  __shared__ int bins[SORT_BINS];
  __shared__ int partial[1024];
  // workgroup t * windows + w orders bags w * window .. of table t among themselves
  const int windows = (B_table + window - 1) / window;
  const int t = blockIdx.x / windows;
  const int tid = threadIdx.x;
  const int first = (blockIdx.x - t * windows) * window;
  const int B = B_table - first < window ? B_table - first : window;
  const int64_t ob = (int64_t)t * B_table + first;
  for (int i = tid; i < SORT_BINS; i += 1024) bins[i] = 0;
  __syncthreads();
  // bin of a bag: SORT_BINS - 1 - min(length, SORT_BINS - 1), so that the longest come first
  // the first two bags of every thread stay in registers between the two passes
  int64_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;
  for (int b = tid, it = 0; b < B; b += 1024, ++it) {
    const int64_t o0 = read_offset(offsets, off64, ob + b), o1 = read_offset(offsets, off64, ob + b + 1);
    if (it == 0) {
      a0 = o0;
      a1 = o1;
    } else if (it == 1) {
      b0 = o0;
      b1 = o1;
    }
    int64_t len = o1 - o0;
    len = len < 0 ? 0 : (len > SORT_BINS - 1 ? SORT_BINS - 1 : len);
    atomicAdd(&bins[SORT_BINS - 1 - (int)len], 1);
  }
  __syncthreads();
  // exclusive scan of the SORT_BINS (== blockDim) counters: inside each wave
  // through lane shuffles, then over the 16 wave totals
  const int mine = bins[tid];
  int incl = mine;
  const int lane = tid & 63;
  for (int step = 1; step < 64; step <<= 1) {
    const int v = __shfl_up(incl, step, 64);
    if (lane >= step) incl += v;
  }
  if (lane == 63) partial[tid >> 6] = incl;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < (tid >> 6); ++w) before += partial[w];
  bins[tid] = before + incl - mine;
  __syncthreads();
  for (int b = tid, it = 0; b < B; b += 1024, ++it) {
    int64_t o0, o1;
    if (it == 0) {
      o0 = a0;
      o1 = a1;
    } else if (it == 1) {
      o0 = b0;
      o1 = b1;
    } else {
      o0 = read_offset(offsets, off64, ob + b);
      o1 = read_offset(offsets, off64, ob + b + 1);
    }
    const int64_t exact = o1 - o0;
    const int64_t len = exact < 0 ? 0 : (exact > SORT_BINS - 1 ? SORT_BINS - 1 : exact);
    const int p = atomicAdd(&bins[SORT_BINS - 1 - (int)len], 1);
    BagEntry be;
    be.o0 = o0;
    be.len = (exact < 0 || exact > 0x7fffffffLL) ? -1 : (int32_t)exact;
    be.bag = first + b;
    order[ob + p] = be;
  }
}

// ---- helpers ----------------------------------------------------------------

// lengths -> offsets (exclusive prefix sum), one workgroup. Used when the
// caller passes Caffe2-style lengths instead of offsets.
template <typename T>
__global__ __launch_bounds__(1024) void lengths_to_offsets_kernel(const T* lengths, int64_t n, int64_t* offsets) {
  __shared__ int64_t part[1024];
  const int tid = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = (int64_t)tid * per;
  const int64_t hi = lo + per < n ? lo + per : n;
  int64_t sum = 0;
  for (int64_t i = lo; i < hi; ++i) sum += (int64_t)(int)lengths[i];
  part[tid] = sum;
  __syncthreads();
  for (int step = 1; step < 1024; step <<= 1) {
    int64_t v = tid >= step ? part[tid - step] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int64_t run = part[tid] - sum;
  for (int64_t i = lo; i < hi; ++i) {
    offsets[i] = run;
    run += (int64_t)(int)lengths[i];
  }
  if (tid == 1023) offsets[n] = part[1023];
}

__global__ void status_clear_kernel(Status* st) {
  st->bits = 0;
  st->pad = 0;
  st->first_bad_pos = ~0ull;
}

// dense[i] = remap[remap_offsets[t] + idx[i]] for tables with a mapping, a copy
// otherwise (…/embedding_forward_quantized_cpu_template.cpp:605-659).
template <typename index_t, typename remap_t>
__global__ __launch_bounds__(256) void pruned_array_lookup_kernel(
    const index_t* indices, const index_t* offsets, const remap_t* remap,
    const int64_t* remap_offsets, int32_t B, int32_t T, index_t* dense) {
  const int t = blockIdx.y;
  const int64_t rs = remap_offsets[t], re = remap_offsets[t + 1];
  const int64_t is = offsets[(int64_t)t * B], ie = offsets[(int64_t)(t + 1) * B];
  const bool mapped = re - rs > 0;
  for (int64_t i = is + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < ie; i += (int64_t)gridDim.x * blockDim.x) {
    index_t v = indices[i];
    // an id outside the mapping reads nothing (the reference reads out of bounds there)
    if (mapped) v = (v >= 0 && (int64_t)v < re - rs) ? (index_t)remap[rs + v] : (index_t)-1;
    dense[i] = v;
  }
}

// ---- launchers (called from the C ABI) ---------------------------------------

hipError_t launch_lookup_i64(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_i32(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_i64_general(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_i32_general(const LookupArgs& a, unsigned blocks, hipStream_t stream);

hipError_t launch_lookup_lean_i64_exact(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_exact(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i64_fast(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_fast(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i64_exact_w4(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_exact_w4(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i64_fast_w4(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_fast_w4(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i64_exact_q8(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_exact_q8(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i64_fast_q8(const LookupArgs& a, unsigned blocks, hipStream_t stream);
hipError_t launch_lookup_lean_i32_fast_q8(const LookupArgs& a, unsigned blocks, hipStream_t stream);

// The lean kernel (lookup_lean.h) over a work list (or a single table) whose tables all
// have a lean shape. `exact` selects the reference's sequence of roundings; `wide4`: every table
// of the launch has the shape lookup_lean_wide4_kernel takes.
hipError_t launch_lookup_lean(const LookupArgs& a, bool idx64, bool exact, bool wide4, hipStream_t stream) {
  if (a.num_waves <= 0) return hipSuccess;
  const int64_t blocks = a.xcd_start ? 8 * a.num_waves : a.num_waves;
  if (blocks > 0x7fffffffLL || a.positional) return hipErrorInvalidValue;
  if (a.out_ty == ST_INT8) { // the instances whose output stage quantizes the pooled vectors (lean_store_q8)
    if (exact) return idx64 ? launch_lookup_lean_i64_exact_q8(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_exact_q8(a, (unsigned)blocks, stream);
    return idx64 ? launch_lookup_lean_i64_fast_q8(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_fast_q8(a, (unsigned)blocks, stream);
  }
  if (wide4) { // two launches: the kernel, and the one that pools what it has queued
    if (!a.redo || !a.redo_count || !a.tables) return hipErrorInvalidValue;
    if (exact) return idx64 ? launch_lookup_lean_i64_exact_w4(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_exact_w4(a, (unsigned)blocks, stream);
    return idx64 ? launch_lookup_lean_i64_fast_w4(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_fast_w4(a, (unsigned)blocks, stream);
  }
  if (exact) return idx64 ? launch_lookup_lean_i64_exact(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_exact(a, (unsigned)blocks, stream);
  return idx64 ? launch_lookup_lean_i64_fast(a, (unsigned)blocks, stream) : launch_lookup_lean_i32_fast(a, (unsigned)blocks, stream);
}

hipError_t launch_lookup(const LookupArgs& a, bool idx64, hipStream_t stream) {
  if (a.num_waves <= 0) return hipSuccess;
  const int64_t blocks = a.xcd_start ? 8 * a.num_waves : a.num_waves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool general = a.remap || a.positional || a.check_total;
  if (general) return idx64 ? launch_lookup_i64_general(a, (unsigned)blocks, stream) : launch_lookup_i32_general(a, (unsigned)blocks, stream);
  return idx64 ? launch_lookup_i64(a, (unsigned)blocks, stream) : launch_lookup_i32(a, (unsigned)blocks, stream);
}

hipError_t launch_bag_order(const void* offsets, bool off64, int32_t B, int32_t T, BagEntry* order, hipStream_t stream) {
  if (T <= 0 || B <= 0) return hipSuccess;
  // Tables of up to SORT_WHOLE_TABLE bags are ordered as a whole: their launches are a few rounds of
  // waves, and longest-first over the whole table is what keeps the drain of such a launch short
  // (32 tables x 4 096 bags of 5..50 rows: 88 us ordered whole, 100 us in windows of 2 048).
  const int window = B <= SORT_WHOLE_TABLE ? B : SORT_WINDOW;
  const int64_t blocks = (int64_t)((B + window - 1) / window) * T;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(bag_order_kernel, dim3((unsigned)blocks), dim3(1024), 0, stream, offsets, off64 ? 1 : 0, B, window, order);
  return hipGetLastError();
}

hipError_t launch_lengths_to_offsets(const void* lengths, bool is64, int64_t n, int64_t* offsets, hipStream_t stream) {
  if (is64) hipLaunchKernelGGL(lengths_to_offsets_kernel<int64_t>, dim3(1), dim3(1024), 0, stream, (const int64_t*)lengths, n, offsets);
  else hipLaunchKernelGGL(lengths_to_offsets_kernel<int32_t>, dim3(1), dim3(1024), 0, stream, (const int32_t*)lengths, n, offsets);
  return hipGetLastError();
}

hipError_t launch_status_clear(Status* st, hipStream_t stream) {
  hipLaunchKernelGGL(status_clear_kernel, dim3(1), dim3(1), 0, stream, st);
  return hipGetLastError();
}

hipError_t launch_pruned_array_lookup(const void* indices, const void* offsets, bool idx64, const void* remap,
                                      bool remap64, const int64_t* remap_offsets, int32_t B, int32_t T,
                                      void* dense, hipStream_t stream) {
  if (T <= 0 || B <= 0) return hipSuccess;
  dim3 grid(64, (unsigned)T), block(256);
  if (idx64 && remap64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int64_t, int64_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int64_t*)remap, remap_offsets, B, T, (int64_t*)dense);
  else if (idx64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int64_t, int32_t>), grid, block, 0, stream, (const int64_t*)indices, (const int64_t*)offsets, (const int32_t*)remap, remap_offsets, B, T, (int64_t*)dense);
  else if (remap64)
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int32_t, int64_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int64_t*)remap, remap_offsets, B, T, (int32_t*)dense);
  else
    hipLaunchKernelGGL((pruned_array_lookup_kernel<int32_t, int32_t>), grid, block, 0, stream, (const int32_t*)indices, (const int32_t*)offsets, (const int32_t*)remap, remap_offsets, B, T, (int32_t*)dense);
  return hipGetLastError();
}

} // namespace fbgemm_amd
