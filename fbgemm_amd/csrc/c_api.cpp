// Host side of the C ABI declared in include/fbgemm_amd.h: argument checks,
// per-table lane mapping, work lists, launches. No torch types here.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "../../include/fbgemm_amd.h"
#include "../../include/fbgemm_amd_bench.h"
#include "cache_policy.h"
#include "lookup_common.h"

#include "launchers.h"

using namespace fbgemm_amd;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(expr)                                                                   \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess) return fail(FBGEMM_AMD_E_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

int type_bits(int ty) {
  switch (ty) {
    case ST_FP32: return 32;
    case ST_FP16: case ST_BF16: return 16;
    case ST_INT8: case ST_FP8: return 8;
    case ST_INT4: return 4;
    case ST_INT2: return 2;
    default: return 0;
  }
}

bool quantised(int ty) { return ty == ST_INT8 || ty == ST_INT4 || ty == ST_INT2; }

int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : dflt;
}

// Tunables, read once per process (the reference reads its FBGEMM_* switches
// the same way, src/Utils.cc:773-875).

constexpr int64_t SORT_MIN_LOOKUPS = 1 << 21;

// 1: order each table's bags by length on the device before the lookup.
int sort_bags_default() {
  static int v = env_int("FBGEMM_AMD_SORT_BAGS", 1);
  return v;
}

// Choose how lanes split a row. Wide 16-byte lanes need every row's data and
// scale/bias to sit on 4-byte boundaries; anything else falls back to 4-byte
// lanes and finally to element-sized lanes, which accept any layout.
// `narrow`: 4-byte lanes where 16-byte ones would do. More lanes per bag means fewer bags per
// wave and more waves: a launch too small to fill the device is bound by the chain of memory
// round trips inside a wave, and spreading its bags over more waves shortens nothing per wave but
// lets every compute unit work (measured: the 1 024-bag 8-bit table 13.0 -> 9.7 us, the 4 096-bag
// 4-bit table 22.8 -> 15.8 us; rounds of 16 rows on top of that changed nothing).
void plan_lanes(TableDesc& d, uintptr_t base_addr, int64_t out_stride, bool has_sb, bool allow_packed, bool narrow = false) {
  const int bits = type_bits(d.ty);
  d.data_bytes = (int32_t)(((int64_t)d.D * bits + 7) / 8);
  const bool a4 = base_addr % 4 == 0 && d.weights_offset % 4 == 0 && d.row_stride % 4 == 0 &&
      d.data_off % 4 == 0 && (!has_sb || d.sb_off % 4 == 0);
  const int min_vb = bits >= 16 ? bits / 8 : 1;
  int vb = min_vb;
  if (a4 && d.data_bytes % 16 == 0 && d.ty != ST_INT2) vb = 16;
  else if (a4 && d.data_bytes % 4 == 0) vb = 4;
  if (narrow && vb == 16) vb = 4;
  d.vb = vb;
  const int chunks = (d.data_bytes + vb - 1) / vb;
  // Wide rows: give a lane several 16-byte chunks (up to 32 accumulators), so
  // that the per-row bookkeeping is shared by more elements.
  const int type_c = bits >= 16 ? 4 : (bits == 8 ? 2 : 1);
  int C = 1;
  if (vb == 16)
    for (int c = type_c; c > 1; c >>= 1)
      if (chunks % c == 0 && chunks / c >= 2) { C = c; break; }
  d.chunks = C;
  d.lanes = std::max(2, std::min(64, chunks / C)); // >= 2: a wave stages at most 32 bags
  d.passes = (chunks + d.lanes * C - 1) / (d.lanes * C);
  // Whole-row chunks for 4- and 8-bit rows with the fp16 header first and a
  // stride that is a multiple of 16: the header rides in chunk 0 and costs no
  // memory request of its own. Needs every 16-byte load of a row to stay
  // inside the row's stride and a single pass.
  d.inline_hdr = 0;
  if (has_sb && (d.ty == ST_INT4 || d.ty == ST_INT8) && !d.sb_fp32 && d.sb_off == 0 && d.data_off == 4 &&
      base_addr % 16 == 0 && d.weights_offset % 16 == 0 && d.row_stride % 16 == 0 && !narrow) {
    const int nchunks = (d.data_bytes + 4 + 15) / 16;
    const int Ci = (d.ty == ST_INT8 && nchunks >= 4) ? 2 : 1;
    const int lanes = std::max(2, (nchunks + Ci - 1) / Ci);
    // lanes that would idle because a bag may not straddle a quarter of the wave:
    // too many (9 lanes per bag) and the bags are laid end to end instead
    const int used = lanes <= 16 ? (16 / lanes) * lanes : 16;
    const bool pack = used < 14 && allow_packed && (64 / lanes) * lanes >= 56;
    if (lanes <= 32 && (int64_t)nchunks * 16 <= d.row_stride && (used >= 14 || pack)) {
      d.inline_hdr = 1;
      d.packed = pack ? 1 : 0;
      d.vb = 16;
      d.chunks = Ci;
      d.lanes = lanes;
      d.passes = 1;
      // runs of E / 4 columns, each stored whole when aligned
      const int GE = (16 * 8 / bits) / 4;
      d.vec_store = 0;
      for (int k = 0; k < 2; ++k) {
        const int esz = k == 0 ? 4 : 2;
        const int al = std::min(16, GE * esz);
        if ((out_stride * esz) % al == 0 && ((int64_t)d.out_col * esz) % al == 0) d.vec_store |= 1 << k;
      }
      return;
    }
  }
  // whole-run vector stores: each lane writes E = vb*8/bits consecutive
  // elements; allowed when every run starts on a multiple of min(16, run bytes)
  // and no run is cut by the end of the row.
  const int E = vb * 8 / bits;
  d.vec_store = 0;
  if (d.D % E == 0) {
    for (int k = 0; k < 2; ++k) {
      const int esz = k == 0 ? 4 : 2;
      const int run = E * esz;
      const int al = std::min(16, run);
      if ((run == 2 || run == 4 || run == 8 || run % 16 == 0) && (out_stride * esz) % al == 0 &&
          ((int64_t)d.out_col * esz) % al == 0)
        d.vec_store |= 1 << k;
    }
  }
}

// What fetching one row costs, in 128-byte line requests (what the memory
// system charges for): the lines the loaded bytes of a row touch, averaged over
// the alignments rows of this stride take, plus a request for a scale/bias pair
// that is fetched apart from the data, plus the row's share of the index,
// weight and bookkeeping traffic (fitted to measured run times: about a third
// of a line).
double row_cost(const TableDesc& d) {
  const bool q = quantised(d.ty);
  int64_t first = 0, last; // bytes of the row that are loaded: [first, last)
  if (d.inline_hdr) {
    last = ((int64_t)d.data_bytes + 4 + 15) / 16 * 16;
  } else {
    first = d.data_off;
    last = (int64_t)d.data_off + d.data_bytes;
    if (q) {
      first = std::min<int64_t>(first, d.sb_off);
      last = std::max<int64_t>(last, (int64_t)d.sb_off + (d.sb_fp32 ? 8 : 4));
    }
  }
  // rows start at (offset of row 0 + k * gcd(stride, 128)) mod 128
  int64_t g = 128, b = d.row_stride % 128;
  while (b) { const int64_t r = g % b; g = b; b = r; }
  double lines = 0;
  for (int64_t k = 0; k < 128 / g; ++k) {
    const int64_t o = (d.weights_offset % 128 + k * g) % 128;
    lines += (double)((o + last - 1) / 128 - (o + first) / 128 + 1);
  }
  lines /= (double)(128 / g);
  if (q && !d.inline_hdr) lines += 0.5;
  if (d.packed) lines += 0.4; // bags that straddle a quarter of the wave ask for some lines twice
  return lines + 0.35;
}

// Launches of fewer waves than this take 4-byte lanes (see plan_lanes). Read once; tests set it.
int g_narrow_override = -1;
int narrow_below_waves() {
  static int v = env_int("FBGEMM_AMD_NARROW_BELOW_WAVES", 1024);
  return g_narrow_override >= 0 ? g_narrow_override : v;
}

// 1: shapes the lean kernel takes go to it (0: everything through the general kernel, for A/B runs and tests).
int lean_default() {
  static int v = env_int("FBGEMM_AMD_LEAN", 1);
  return v;
}
int g_lean_override = -1; // tests: fbgemm_amd_set_lean

bool lean_enabled() { return g_lean_override >= 0 ? g_lean_override != 0 : lean_default() != 0; }

// What lookup_lean.h pools: 4-bit / 8-bit / fp16 rows read as 16-byte chunks at 4-byte
// alignment in one pass, every lane owning 32 columns (1 / 2 / 4 chunks), rows numbered in 31 bits.
bool lean_shape(const TableDesc& d) {
  const int want_c = d.ty == ST_INT4 ? 1 : d.ty == ST_INT8 ? 2 : d.ty == ST_FP16 ? 4 : 0;
  if (!want_c || d.vb != 16 || d.passes != 1 || d.chunks != want_c) return false;
  if (d.lanes < 2 || d.lanes > 64) return false;
  if (d.num_rows > (1LL << 31) || d.row_stride <= 0 || d.row_stride > 0xffffffffLL) return false;
  if (!d.inline_hdr && (int64_t)d.lanes * d.chunks * 16 != d.data_bytes) return false;
  return true;
}

// Shapes of the lean kernel's four-waves-per-SIMD instance (lookup_lean_wide4_kernel): 4-bit rows,
// bags of 8 lanes and more (one entry per staging lane), the header fetched by a staging lane.
bool lean_wide4_shape(const TableDesc& d) {
  return lean_shape(d) && d.ty == ST_INT4 && d.lanes >= 8 && !d.inline_hdr;
}
// When forwards that could take that instance do: 0 never, 2 always, 1 (default) whichever of
// the two kernels the first forwards of a work set measure as the faster one (FBGEMM_AMD_WIDE4 at
// load time; fbgemm_amd_set_wide4 for tests and benchmarks).
int g_wide4_override = -1;
int wide4_mode() {
  static const int dflt = env_int("FBGEMM_AMD_WIDE4", 1);
  const int m = g_wide4_override >= 0 ? g_wide4_override : dflt;
  return m < 0 ? 0 : (m > 2 ? 2 : m);
}

struct DeviceScratch {
  Status* status = nullptr;
  int64_t* offsets = nullptr; // lengths -> offsets
  int64_t offsets_cap = 0;
  BagEntry* order = nullptr;  // bag order of single-table calls
  int64_t order_cap = 0;
  int64_t* fixed = nullptr;   // bounds check: repaired offsets before they are written back
  int64_t fixed_cap = 0;
  int64_t* partial = nullptr; // bounds check: per-block maxima of the offset scan
  int64_t partial_cap = 0;
  int64_t* seg_offsets = nullptr; // split bags: where every segment starts
  int64_t seg_offsets_cap = 0;
  float* seg_partial = nullptr;   // split bags: the segments' fp32 sums
  int64_t seg_partial_cap = 0;
};

// Few, long bags (tolerance-grade accumulate only): the number of segments a bag is cut into so that
// the launch has enough waves to fill the device. `waves` = what the launch would have, `avg_len` =
// entries per bag on average. 1 = no split.
int split_factor(int64_t waves, int64_t avg_len) {
  static const int enabled = env_int("FBGEMM_AMD_SPLIT_BAGS", 1);
  if (!enabled || waves >= 256 || avg_len < 32) return 1;
  int K = 2;
  while (K < 32 && K * 2 * 8 <= avg_len && waves * K < 1024) K *= 2; // segments of 8 rows at least
  return K;
}

// Grow-only device buffer; the old one may still be read by an enqueued kernel.
template <typename T>
int grow(T** buf, int64_t* cap, int64_t need, hipStream_t stream);

std::mutex& g_mu = *new std::mutex();

// The status block and scratch buffers behind the calls that own their scratch
// (fbgemm_amd_spmdm_run, the lengths / bag-order / split-bag buffers of fbgemm_amd_spmdm_launch,
// bounds checks, pruning): one set per host thread and device, so that threads calling
// concurrently, each on a stream of its own, neither read each other's status bits nor free a
// buffer another thread's enqueued kernel still uses. A thread that ends hands its sets to
// g_idle_scratch (no HIP call at thread exit); the next new thread adopts one after a device-wide
// synchronize. Calls of ONE thread share its set: those must be ordered on one stream.
// (The map and the mutex are never destroyed: threads may end, and hand their sets over, while the
// process runs its static destructors. What the sets hold stays allocated until the process ends.)
std::map<int, std::vector<DeviceScratch>>& g_idle_scratch = *new std::map<int, std::vector<DeviceScratch>>(); // guarded by g_mu

struct ThreadScratch {
  std::map<int, DeviceScratch> by_device;
  ~ThreadScratch() {
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto& kv : by_device)
      if (kv.second.status) g_idle_scratch[kv.first].push_back(kv.second);
  }
};
thread_local ThreadScratch t_scratch;

// call with g_mu held
int get_scratch(DeviceScratch** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  DeviceScratch& s = t_scratch.by_device[dev];
  if (!s.status) {
    std::vector<DeviceScratch>& idle = g_idle_scratch[dev];
    if (!idle.empty()) {
      HIP_TRY(hipDeviceSynchronize()); // what its last owner enqueued has finished
      s = idle.back();
      idle.pop_back();
    } else {
      HIP_TRY(hipMalloc((void**)&s.status, sizeof(Status)));
    }
  }
  *out = &s;
  return 0;
}

template <typename T>
int grow(T** buf, int64_t* cap, int64_t need, hipStream_t stream) {
  if (*cap >= need) return 0;
  HIP_TRY(hipStreamSynchronize(stream));
  HIP_TRY(hipDeviceSynchronize());
  if (*buf) HIP_TRY(hipFree(*buf));
  *buf = nullptr;
  *cap = 0;
  const int64_t n = std::max<int64_t>(need + need / 2, 4096);
  HIP_TRY(hipMalloc((void**)buf, sizeof(T) * n));
  *cap = n;
  return 0;
}

int check_cfg(const fbgemm_amd_spmdm_config* c) {
  if (!c) return fail(FBGEMM_AMD_E_ARG, "config is null");
  if (type_bits(c->weight_ty) == 0) return fail(FBGEMM_AMD_E_ARG, "unsupported weight_ty %d", c->weight_ty);
  if (c->weight_ty == ST_FP8 &&
      (c->fp8_exponent_bits < 1 || c->fp8_exponent_bits > 6 || c->fp8_exponent_bias < 0 || c->fp8_exponent_bias > 253))
    return fail(FBGEMM_AMD_E_ARG, "fp8 rows need 1..6 exponent bits and a bias in 0..253");
  const bool float_out = c->output_ty == ST_FP32 || c->output_ty == ST_FP16 || c->output_ty == ST_BF16;
  if (c->no_bag) {
    // the combinations the reference has (src/RefImplementations.cc:1235-1288,1352-1376,1466-1484)
    if (c->weight_ty == ST_INT4 ? c->output_ty != ST_INT4
                                : (c->weight_ty == ST_INT2 || c->weight_ty == ST_FP8 ||
                                   !(float_out || (c->weight_ty == ST_INT8 && c->output_ty == ST_INT8))))
      return fail(FBGEMM_AMD_E_ARG, "no_bag: weight_ty %d has no output_ty %d", c->weight_ty, c->output_ty);
  } else if (!float_out) {
    return fail(FBGEMM_AMD_E_ARG, "unsupported output_ty %d", c->output_ty);
  }
  if ((c->index_bits != 32 && c->index_bits != 64) || (c->offset_bits != 32 && c->offset_bits != 64))
    return fail(FBGEMM_AMD_E_ARG, "index_bits/offset_bits must be 32 or 64");
  if (c->block_size <= 0 || c->block_size > (1 << 24)) return fail(FBGEMM_AMD_E_ARG, "bad block_size");
  if (c->accumulate != FBGEMM_AMD_ACC_EXACT && c->accumulate != FBGEMM_AMD_ACC_FAST)
    return fail(FBGEMM_AMD_E_ARG, "accumulate must be FBGEMM_AMD_ACC_EXACT or FBGEMM_AMD_ACC_FAST");
  return 0;
}

} // namespace

extern "C" {

const char* fbgemm_amd_last_error(void) { return g_err; }
const char* fbgemm_amd_version(void) { return "0.1"; }

int fbgemm_amd_status_clear(void* d_status, void* stream) {
  if (!d_status) return fail(FBGEMM_AMD_E_ARG, "d_status is null");
  HIP_TRY(launch_status_clear((Status*)d_status, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_status_read(const void* d_status, void* stream, int32_t* bits, int64_t* first_bad_pos) {
  if (!d_status) return fail(FBGEMM_AMD_E_ARG, "d_status is null");
  Status h;
  HIP_TRY(hipMemcpyAsync(&h, d_status, sizeof(h), hipMemcpyDeviceToHost, (hipStream_t)stream));
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  if (bits) *bits = h.bits;
  if (first_bad_pos) *first_bad_pos = h.first_bad_pos == ~0ull ? -1 : (int64_t)h.first_bad_pos;
  return 0;
}

int fbgemm_amd_stream_synchronize(void* stream) {
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}

int32_t fbgemm_amd_unpadded_row_size_in_bytes(int32_t dim, int32_t ty, int32_t sb) {
  switch (ty) {
    case ST_FP32: return dim * 4;
    case ST_FP16: case ST_BF16: return dim * 2;
    case ST_FP8: return dim;
    case ST_INT8: return dim + sb;
    case ST_INT4: return dim / 2 + sb;
    case ST_INT2: return dim / 4 + sb;
    default: return 0;
  }
}

int32_t fbgemm_amd_padded_row_size_in_bytes(int32_t dim, int32_t ty, int32_t row_alignment, int32_t sb) {
  const uint64_t r = (uint64_t)fbgemm_amd_unpadded_row_size_in_bytes(dim, ty, sb);
  const uint64_t a = (uint64_t)(row_alignment > 0 ? row_alignment : 1);
  return (int32_t)((r + a - 1) / a * a);
}

} // extern "C"

namespace {

// ---- scratch of the entry point that allocates nothing ------------------------
//
// fbgemm_amd_spmdm_launch_noalloc keeps what fbgemm_amd_spmdm_launch would put
// into hipMalloc'ed scratch (the prefix sum of Caffe2-style lengths, the bag
// order of the scheduler) in this array, which is part of the code object:
// every GPU the library runs on holds its own copy from module load until the
// process ends. Host code never uses the array's name as an address; the
// device address is asked for once per device (noalloc_scratch_ptr).
constexpr int64_t NOALLOC_MAX_BAGS = FBGEMM_AMD_NOALLOC_MAX_BAGS;
constexpr size_t NOALLOC_OFFSETS_BYTES = ((size_t)(NOALLOC_MAX_BAGS + 1) * sizeof(int64_t) + 255) / 256 * 256;
constexpr size_t NOALLOC_ORDER_BYTES = (size_t)NOALLOC_MAX_BAGS * sizeof(BagEntry);
static __device__ __align__(256) unsigned char scratch[NOALLOC_OFFSETS_BYTES + NOALLOC_ORDER_BYTES];

std::map<int, unsigned char*> g_noalloc_ptr; // per device; guarded by g_mu

// Device address of the current device's copy of `scratch`. Allocates nothing:
// the array came with the code object.
int noalloc_scratch_ptr(unsigned char** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_noalloc_ptr.find(dev);
  if (it == g_noalloc_ptr.end()) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(FBGEMM_AMD_E_HIP, "hipGetSymbolAddress gave no address for the static scratch array");
    it = g_noalloc_ptr.emplace(dev, (unsigned char*)p).first;
  }
  *out = it->second;
  return 0;
}

int spmdm_launch_impl(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_remap, void* d_status, void* stream_, bool noalloc) {
  if (int rc = check_cfg(cfg)) return rc;
  if (noalloc && output_size > NOALLOC_MAX_BAGS)
    return fail(FBGEMM_AMD_E_ARG, "fbgemm_amd_spmdm_launch_noalloc takes at most %lld bags per call (got %lld); "
                "use fbgemm_amd_spmdm_launch", (long long)NOALLOC_MAX_BAGS, (long long)output_size);
  if (!d_status) return fail(FBGEMM_AMD_E_ARG, "d_status is null");
  if (output_size < 0 || index_size < 0 || data_size < 0) return fail(FBGEMM_AMD_E_ARG, "negative size");
  if (output_size > 0x7fffffffLL) return fail(FBGEMM_AMD_E_ARG, "output_size exceeds 2^31-1");
  hipStream_t stream = (hipStream_t)stream_;
  if (output_size == 0) {
    // the reference returns (0 == index_size) without touching anything
    if (index_size != 0 && !cfg->no_bag) {
      Status h{ERR_LENGTH_MISMATCH, 0, ~0ull};
      HIP_TRY(hipMemcpyAsync(d_status, &h, sizeof(h), hipMemcpyHostToDevice, stream));
      HIP_TRY(hipStreamSynchronize(stream));
    }
    return 0;
  }
  if (!d_input || !d_out || (!cfg->no_bag && !d_offsets_or_lengths) || ((index_size > 0 || cfg->no_bag) && !d_indices))
    return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  if (cfg->no_bag && d_remap) return fail(FBGEMM_AMD_E_ARG, "no_bag has no row-wise-sparse variant");
  if (d_remap && !cfg->scale_bias_last && quantised(cfg->weight_ty))
    return fail(FBGEMM_AMD_E_ARG, "row-wise-sparse lookups use the scale_bias_last layout");
  if (d_remap && cfg->output_ty != ST_FP32)
    return fail(FBGEMM_AMD_E_ARG, "row-wise-sparse lookups write fp32");

  const int ty = cfg->weight_ty;
  const int bits = type_bits(ty);
  const int64_t D = cfg->block_size;
  const int64_t elem_bytes = bits >= 8 ? bits / 8 : 1; // storage element of input_stride
  LookupArgs a;
  memset(&a, 0, sizeof(a));
  TableDesc& d = a.single;
  d.ty = ty;
  d.D = (int32_t)D;
  d.out_col = 0;
  d.num_rows = data_size;
  d.placement = 0;
  d.weights_offset = 0;
  d.skip_minus_one = cfg->scale_bias_last ? 0 : 1;
  bool has_sb = false;
  if (quantised(ty)) {
    has_sb = true;
    const int64_t packed = (D * bits + 7) / 8;
    const int64_t sb = (ty == ST_INT8 && cfg->scale_bias_last) ? 8 : 4;
    d.sb_fp32 = sb == 8;
    d.row_stride = cfg->input_stride == -1 ? packed + sb : cfg->input_stride;
    if (cfg->scale_bias_last) {
      d.data_off = 0;
      d.sb_off = (int32_t)packed;
    } else {
      d.sb_off = 0;
      d.data_off = (int32_t)sb;
    }
  } else {
    d.row_stride = (cfg->input_stride == -1 ? D : cfg->input_stride) * elem_bytes;
    d.data_off = 0;
    d.sb_off = 0;
  }
  const int64_t out_stride = cfg->output_stride == -1 ? D : cfg->output_stride;
  if ((ty == ST_FP16 || ty == ST_BF16) && (uintptr_t)d_input % 2) return fail(FBGEMM_AMD_E_ARG, "fp16 table must be 2-byte aligned");
  if (ty == ST_FP32 && (uintptr_t)d_input % 4) return fail(FBGEMM_AMD_E_ARG, "fp32 table must be 4-byte aligned");
  if (ty == ST_FP8) {
    a.fp8_shift = 16 + cfg->fp8_exponent_bits;
    const uint32_t mult_bits = (uint32_t)(127 + (127 - cfg->fp8_exponent_bias)) << 23; // 2^(127 - bias)
    memcpy(&a.fp8_mult, &mult_bits, 4);
    d.skip_minus_one = 0; // EmbeddingSpMDMFP8_ref has no pruned-row skip (src/RefImplementations.cc:1584-1587)
  }
  if (cfg->no_bag) {
    // one output row per index; the reference reads exactly output_size indices
    d.data_bytes = (int32_t)((D * bits + 7) / 8);
    int64_t out_stride_bytes, copy_bytes = 0;
    if (ty == ST_INT4) {
      copy_bytes = d.row_stride;
      out_stride_bytes = d.row_stride;
    } else if (cfg->output_ty == ST_INT8) {
      copy_bytes = std::min(out_stride, d.row_stride);
      out_stride_bytes = out_stride;
    } else {
      out_stride_bytes = out_stride * (cfg->output_ty == ST_FP32 ? 4 : 2);
      if ((uintptr_t)d_out % (cfg->output_ty == ST_FP32 ? 4 : 2)) return fail(FBGEMM_AMD_E_ARG, "output is not aligned to its elements");
    }
    if (ty == ST_FP16 || ty == ST_BF16 || ty == ST_FP32) {
      if (d.row_stride % (bits / 8)) return fail(FBGEMM_AMD_E_ARG, "rows are not aligned to their elements");
    }
    HIP_TRY(launch_row_lookup(d, (const uint8_t*)d_input, d_indices, cfg->index_bits == 64, d_weights, output_size,
                              cfg->output_ty, d_out, out_stride_bytes, copy_bytes, a.fp8_shift, a.fp8_mult,
                              (Status*)d_status, stream));
    return 0;
  }
  plan_lanes(d, (uintptr_t)d_input, out_stride, has_sb, false);
  // few, long bags, and the caller accepts sums in another order: cut every bag into K segments.
  // 4- and 8-bit rows only: every other row type is summed the reference's way in either mode,
  // in one piece.
  int K = 1;
  if (!noalloc && cfg->accumulate == FBGEMM_AMD_ACC_FAST && !cfg->is_weight_positional && output_size * 32 <= 0x7fffffffLL &&
      (ty == ST_INT4 || ty == ST_INT8)) {
    const int G16 = bags_per_wave(d.lanes, d.packed);
    K = split_factor((output_size + G16 - 1) / G16, index_size / output_size);
  }
  const int64_t pooled_bags = output_size * K;       // what the lookup kernel sees as bags
  const int64_t pooled_stride = K > 1 ? D : out_stride; // segments' sums are rows of D floats
  if (K > 1) plan_lanes(d, (uintptr_t)d_input, pooled_stride, has_sb, false);
  {
    // a launch of fewer than four waves per compute unit: prefer narrow lanes
    const int G16 = bags_per_wave(d.lanes, d.packed);
    if (d.vb == 16 && (pooled_bags + G16 - 1) / G16 < narrow_below_waves()) plan_lanes(d, (uintptr_t)d_input, pooled_stride, has_sb, false, true);
  }
  d.lanes_recip = (65536 + d.lanes - 1) / d.lanes;
  d.bags = bags_per_wave(d.lanes, d.packed);

  a.tables = nullptr;
  a.weights[0] = (const uint8_t*)d_input;
  a.weights[1] = nullptr;
  a.indices = d_indices;
  a.sample_weights = d_weights;
  a.remap = d_remap;
  a.remap_rows = data_size;
  if (d_remap) {
    d.num_rows = 1LL << 31; // the reference does not bound the physical id (RefImplementations.cc:1789-1791); the mapping's int32 entries do
    d.skip_minus_one = 0;
  }
  a.out = d_out;
  a.out_stride = out_stride;
  a.index_size = index_size;
  a.work = nullptr;
  a.B = (int32_t)output_size;
  a.T = 1;
  a.out_ty = cfg->output_ty;
  a.normalize = cfg->normalize_by_lengths;
  a.positional = cfg->is_weight_positional;
  a.check_total = 1;
  a.out_aligned = (uintptr_t)d_out % 16 == 0;
  a.status = (Status*)d_status;
  const int G = bags_per_wave(d.lanes, d.packed);
  a.num_waves = (output_size + G - 1) / G;

  // Ordering the bags pays once several waves' worth of bags and enough lookups exist
  // (the scheduler launch costs 6-8 us and buys ~5 % of the lookup: it pays from a few million lookups on)
  const bool sort = K == 1 && sort_bags_default() && output_size > 2 * G && index_size >= (int64_t)SORT_MIN_LOOKUPS;
  if (cfg->use_offsets) {
    a.offsets = d_offsets_or_lengths;
    a.off64 = cfg->offset_bits == 64;
  }
  if ((!cfg->use_offsets || sort) && noalloc) {
    // the static array: offsets first, then the bag order. Both are written in
    // full (output_size + 1 offsets, output_size entries) before they are read,
    // so what an earlier call left there does not matter.
    unsigned char* base;
    if (int rc = noalloc_scratch_ptr(&base)) return rc;
    if (!cfg->use_offsets) {
      int64_t* offs = reinterpret_cast<int64_t*>(base);
      HIP_TRY(launch_lengths_to_offsets(d_offsets_or_lengths, cfg->offset_bits == 64, output_size, offs, stream));
      a.offsets = offs;
      a.off64 = 1;
    }
    if (sort) {
      BagEntry* order = reinterpret_cast<BagEntry*>(base + NOALLOC_OFFSETS_BYTES);
      HIP_TRY(launch_bag_order(a.offsets, a.off64, (int32_t)output_size, 1, order, stream));
      a.order = order;
    }
  } else if (!cfg->use_offsets || sort) {
    // library-owned scratch: calls that use it must be ordered on one stream
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceScratch* s;
    if (int rc = get_scratch(&s)) return rc;
    if (!cfg->use_offsets) {
      if (int rc = grow(&s->offsets, &s->offsets_cap, output_size + 1, stream)) return rc;
      HIP_TRY(launch_lengths_to_offsets(d_offsets_or_lengths, cfg->offset_bits == 64, output_size, s->offsets, stream));
      a.offsets = s->offsets;
      a.off64 = 1;
    }
    if (sort) {
      if (int rc = grow(&s->order, &s->order_cap, output_size, stream)) return rc;
      HIP_TRY(launch_bag_order(a.offsets, a.off64, (int32_t)output_size, 1, s->order, stream));
      a.order = s->order;
    }
  }
  if (K > 1) {
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceScratch* s;
    if (int rc = get_scratch(&s)) return rc;
    if (int rc = grow(&s->seg_offsets, &s->seg_offsets_cap, pooled_bags + 1, stream)) return rc;
    if (int rc = grow(&s->seg_partial, &s->seg_partial_cap, pooled_bags * D, stream)) return rc;
    HIP_TRY(launch_split_offsets(a.offsets, a.off64, output_size, K, true, index_size, s->seg_offsets, (Status*)d_status, stream));
    LookupArgs v = a;
    v.offsets = s->seg_offsets;
    v.off64 = 1;
    v.order = nullptr;
    v.B = (int32_t)pooled_bags;
    v.out = s->seg_partial;
    v.out_stride = D;
    v.out_ty = ST_FP32;
    v.normalize = 0;
    v.check_total = 0;
    v.out_aligned = 1;
    v.num_waves = (pooled_bags + G - 1) / G;
    if (lean_enabled() && lean_shape(d)) HIP_TRY(launch_lookup_lean(v, cfg->index_bits == 64, false, false, stream));
    else HIP_TRY(launch_lookup(v, cfg->index_bits == 64, stream));
    HIP_TRY(launch_combine_segments(s->seg_partial, D, (int32_t)output_size, K, 1, nullptr, (int32_t)D, a.offsets, a.off64 != 0,
                                    cfg->normalize_by_lengths != 0, d_out, cfg->output_ty, out_stride, stream));
    return 0;
  }
  if (lean_enabled() && !cfg->is_weight_positional && lean_shape(d))
    HIP_TRY(launch_lookup_lean(a, cfg->index_bits == 64, cfg->accumulate != FBGEMM_AMD_ACC_FAST, false, stream));
  else
    HIP_TRY(launch_lookup(a, cfg->index_bits == 64, stream));
  return 0;
}

} // namespace

extern "C" {

int fbgemm_amd_set_narrow_below_waves(int32_t waves) {
  g_narrow_override = waves < 0 ? -1 : waves;
  return 0;
}

int fbgemm_amd_set_wide4(int32_t mode) {
  g_wide4_override = mode < 0 ? -1 : (mode > 2 ? 2 : mode);
  return 0;
}

int fbgemm_amd_set_lean(int32_t on) {
  g_lean_override = on < 0 ? -1 : (on != 0);
  return 0;
}

int fbgemm_amd_spmdm_launch(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_remap, void* d_status, void* stream) {
  return spmdm_launch_impl(cfg, output_size, index_size, data_size, d_input, d_indices, d_offsets_or_lengths,
                           d_weights, d_out, d_remap, d_status, stream, false);
}

int fbgemm_amd_spmdm_launch_noalloc(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_remap, void* d_status, void* stream) {
  return spmdm_launch_impl(cfg, output_size, index_size, data_size, d_input, d_indices, d_offsets_or_lengths,
                           d_weights, d_out, d_remap, d_status, stream, true);
}

int64_t fbgemm_amd_noalloc_max_bags(void) { return NOALLOC_MAX_BAGS; }

int fbgemm_amd_spmdm_run(
    const fbgemm_amd_spmdm_config* cfg, int64_t output_size, int64_t index_size,
    int64_t data_size, const void* d_input, const void* d_indices,
    const void* d_offsets_or_lengths, const float* d_weights, void* d_out,
    const int32_t* d_remap, void* stream) {
  Status* st;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceScratch* s;
    if (int rc = get_scratch(&s)) return rc;
    st = s->status;
  }
  if (int rc = fbgemm_amd_status_clear(st, stream)) return rc;
  if (int rc = fbgemm_amd_spmdm_launch(cfg, output_size, index_size, data_size, d_input, d_indices,
                                      d_offsets_or_lengths, d_weights, d_out, d_remap, st, stream))
    return rc;
  int32_t bits = 0;
  if (int rc = fbgemm_amd_status_read(st, stream, &bits, nullptr)) return rc;
  return bits == 0 ? 1 : 0;
}

} // extern "C"

// ---- table-batched forward ---------------------------------------------------

struct fbgemm_amd_tbe_plan {
  int32_t T = 0;
  int64_t total_D = 0;
  int64_t row_alignment = 16;
  std::vector<TableDesc> tables; // host copy
  TableDesc* d_tables = nullptr;
  int32_t* d_D_offsets = nullptr; // the T + 1 output column offsets, for the 8-bit pooled output
  int32_t max_D = 0;
  float* pooled_tmp = nullptr;    // fp32 [B, total_D] the 8-bit pooled output is quantized from
  int64_t pooled_tmp_cap = 0;
  int64_t* seg_offsets = nullptr; // split bags: where every segment starts (T*B*K + 1)
  int64_t seg_offsets_cap = 0;
  float* seg_partial = nullptr;   // split bags: the segments' fp32 sums [B*K, total_D]
  int64_t seg_partial_cap = 0;
  // pooled_tmp and seg_* are shared by all streams that run forwards of the plan. Forwards that use
  // them are enqueued one at a time (shared_mu), and one on another stream than the last waits on
  // the device for that one's last use (shared_done, recorded behind it): see SharedScratchUse.
  std::mutex shared_mu;
  hipEvent_t shared_done = nullptr;
  hipStream_t shared_stream = nullptr;
  bool shared_used = false;
  // the same tables with bags laid end to end where that saves a request per row
  // (see bags_per_wave); empty when no table has such a shape. Used for long bags.
  std::vector<TableDesc> tables_packed;
  TableDesc* d_tables_packed = nullptr;
  // the same tables with 4-byte lanes (see plan_lanes): for forwards too small to fill the device
  std::vector<TableDesc> tables_narrow;
  TableDesc* d_tables_narrow = nullptr;
  int device = 0;
  // what a forward needs beyond the tables, cached per (B, lane-shape set): the work lists of
  // the two kernels (tables the lean kernel takes, and the rest) and the bag order the scheduler
  // kernel rewrites on every forward. The bag order is scratch, so every stream that runs
  // forwards of the plan gets a buffer of its own (ORDER_SLOTS of them; one is allocated ahead
  // so that a stream met first under capture, where nothing may be allocated, finds one).
  static constexpr int ORDER_SLOTS = 4;
  struct WorkList {
    WaveWork* d_work = nullptr;
    int64_t* d_xcd_start = nullptr;
    int64_t num_waves = 0;
  };
  struct Work {
    WorkList lean, general;
    BagEntry* d_order[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr}; // T*B bags each, rewritten by every forward
    hipStream_t order_stream[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    bool order_claimed[ORDER_SLOTS] = {false, false, false, false};
    // A second stream per slot, with the two events of the fork and the join: a forward with tables
    // for both lookup kernels runs the general kernel there, beside the lean one (made with the
    // slot's first forward outside a capture; without them the two kernels run one after the other)
    hipStream_t side_stream[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t side_fork[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t side_join[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    // the tables on the general kernel's list (the 8-bit pooled output of the lean kernel's tables
    // is written by the lookup itself, these go through the quantizer afterwards)
    int32_t* d_general_tables = nullptr;
    int32_t n_general_tables = 0;
    bool lean_wide4 = false;     // every table of the lean list has the shape of the four-waves-per-SIMD instance
    // that instance's redo queue, one per bag-order buffer (made with it): lean.num_waves work items
    // and two counters that are zero between forwards
    WaveWork* d_redo[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    int32_t* d_redo_count[ORDER_SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    // Which of the two lean kernels the set's forwards take when both can (wide4_mode() == 1):
    // the first forwards outside a capture run them in turn between two events and wait for the
    // second one (eight forwards of a new batch size that synchronize, like the first one, which
    // allocates); the first sample of each kernel is dropped, and after three more of each the
    // faster one stays (a tie goes to the general-purpose kernel, which is one launch less). Both
    // compute the same bits.
    int w4_decided = -1;            // -1: still measuring; 0 / 1: the general-purpose kernel / the four-wave instance
    int w4_seen[2] = {0, 0};        // measurements started, per kernel
    int w4_samples[2] = {0, 0};     // measurements kept
    float w4_ms[2] = {0.0f, 0.0f};  // their sum
    bool w4_busy = false;           // a forward is measuring (one at a time: the two events are the set's)
    hipEvent_t w4_ev[2] = {nullptr, nullptr};
    bool pinned = false;         // used by a forward under stream capture: a graph may hold its pointers
    uint64_t last_use = 0;
  };
  struct WorkKey {
    int32_t B;
    int variant;
    int lean;
    bool operator<(const WorkKey& o) const {
      if (B != o.B) return B < o.B;
      if (variant != o.variant) return variant < o.variant;
      return lean < o.lean;
    }
  };
  std::map<WorkKey, Work> work;
  uint64_t use_clock = 0;
  int32_t accumulate = FBGEMM_AMD_ACC_EXACT;
  // compact form of the pruned-row mappings (fbgemm_amd_tbe_plan_set_index_remappings)
  RankRecord* d_rank_records = nullptr;
  int64_t* d_rank_offsets = nullptr; // T entries: first record of the table, or -1
  // the T + 1 mapping offsets the records were built for (device copy): forwards that use the
  // records bound and slice the mappings with these, whatever offsets they are handed
  int64_t* d_rank_remap_offsets = nullptr;
  const void* rank_source = nullptr; // the mapping array the records were made from
  int32_t rank_bits = 0;
  int32_t rank_tables = 0;           // tables that use the records
  // lane-shape choice of the last forward, per (B, indices_numel >> 16)
  int32_t shape_B = -1;
  int64_t shape_bucket = -1;
  int shape_variant = 0;
  int shape_narrow = -1;
  std::mutex mu;
  // optional timing of the lookup kernel alone: a ring of (start, stop) event pairs
  int32_t fp8_shift = 0; // FP8 rows: set by fbgemm_amd_tbe_plan_set_fp8
  float fp8_mult = 0.0f;
  bool has_fp8 = false;
  bool reuse_order = false; // benchmarks: forwards skip the scheduler and take the last bag order of their stream
};

namespace {

void free_work(fbgemm_amd_tbe_plan::Work& w) {
  for (fbgemm_amd_tbe_plan::WorkList* l : {&w.lean, &w.general}) {
    if (l->d_work) (void)hipFree(l->d_work);
    if (l->d_xcd_start) (void)hipFree(l->d_xcd_start);
    *l = fbgemm_amd_tbe_plan::WorkList();
  }
  for (int k = 0; k < fbgemm_amd_tbe_plan::ORDER_SLOTS; ++k) {
    if (w.d_order[k]) (void)hipFree(w.d_order[k]);
    w.d_order[k] = nullptr;
    if (w.d_redo[k]) (void)hipFree(w.d_redo[k]);
    if (w.d_redo_count[k]) (void)hipFree(w.d_redo_count[k]);
    w.d_redo[k] = nullptr;
    w.d_redo_count[k] = nullptr;
    w.order_claimed[k] = false;
    if (w.side_fork[k]) (void)hipEventDestroy(w.side_fork[k]);
    if (w.side_join[k]) (void)hipEventDestroy(w.side_join[k]);
    if (w.side_stream[k]) (void)hipStreamDestroy(w.side_stream[k]);
    w.side_fork[k] = w.side_join[k] = nullptr;
    w.side_stream[k] = nullptr;
  }
  for (int k = 0; k < 2; ++k) {
    if (w.w4_ev[k]) (void)hipEventDestroy(w.w4_ev[k]);
    w.w4_ev[k] = nullptr;
  }
  if (w.d_general_tables) (void)hipFree(w.d_general_tables);
  w.d_general_tables = nullptr;
  w.n_general_tables = 0;
}

// The per-wave work list of one kernel over the tables `members` (indices into `tables`).
// The list is 8 runs, one per XCD (see lookup_kernel). Tables are cut into slices of waves,
// the slices are dealt to the XCDs so that every XCD gets the same number of 128-byte line
// requests (what the memory system charges for), and inside a run every slice advances
// through its bag order (longest first) at the same relative pace, so that tables of
// different row types share the CUs at all times.
int build_work_list(const std::vector<TableDesc>& tables, const std::vector<int>& members, int32_t B,
                    fbgemm_amd_tbe_plan::WorkList* out) {
  *out = fbgemm_amd_tbe_plan::WorkList();
  if (members.empty()) return 0;
  struct Slice { int t, first, step, count; double cost; };
  std::vector<Slice> slices;
  double total_cost = 0;
  const int T = (int)tables.size();
  std::vector<double> wave_cost(T, 0.0);
  std::vector<int> nwaves(T, 0);
  for (int t : members) {
    const TableDesc& d = tables[t];
    const int G = bags_per_wave(d.lanes, d.packed);
    nwaves[t] = (B + G - 1) / G;
    wave_cost[t] = G * row_cost(d);
    total_cost += wave_cost[t] * nwaves[t];
  }
  const int nx = 8;
  for (int t : members) {
    // slices no larger than 1/4 of an XCD's share; slice p takes waves p, p + parts, ...
    int parts = (int)std::ceil(wave_cost[t] * nwaves[t] / (total_cost / nx / 4.0 + 1e-9));
    parts = std::max(1, std::min(parts, std::min(nwaves[t], nx)));
    for (int p = 0; p < parts; ++p) {
      const int count = (nwaves[t] - p + parts - 1) / parts;
      slices.push_back(Slice{t, p, parts, count, wave_cost[t] * count});
    }
  }
  std::stable_sort(slices.begin(), slices.end(), [](const Slice& x, const Slice& y) { return x.cost > y.cost; });
  std::vector<std::vector<Slice>> per_x(nx);
  std::vector<double> load(nx, 0.0);
  for (const Slice& sl : slices) {
    const int x = (int)(std::min_element(load.begin(), load.end()) - load.begin());
    per_x[x].push_back(sl);
    load[x] += sl.cost;
  }
  std::vector<WaveWork> list;
  std::vector<int64_t> xcd_start(9, 0);
  int64_t longest = 0;
  // Inside a run the slices are walked in groups that hold one slice of every
  // row shape (type, D) the run has; the slices of a group advance together,
  // each through its bag order at the same relative pace, and the groups
  // follow one another. Mixing shapes keeps waves of different cost on the
  // CUs at all times; taking few tables at a time keeps the working set of
  // the XCD's L2 small (hot rows of a table are reused while they are there).
  for (int x = 0; x < nx; ++x) {
    std::vector<std::pair<double, WaveWork>> keyed;
    std::map<std::pair<int, int>, std::vector<Slice>> shapes; // slices of a shape, largest first (per_x order)
    for (const Slice& sl : per_x[x]) {
      const TableDesc& d = tables[sl.t];
      shapes[std::make_pair((int)d.ty, (int)d.D)].push_back(sl);
    }
    size_t depth = 0;
    for (auto& kv : shapes) depth = std::max(depth, kv.second.size());
    int gidx = 0;
    for (size_t i = 0; i < depth; ++i) {
      for (auto& kv : shapes) {
        if (i >= kv.second.size()) continue;
        const Slice& sl = kv.second[i];
        const int G = bags_per_wave(tables[sl.t].lanes, tables[sl.t].packed);
        for (int k = 0; k < sl.count; ++k)
          keyed.push_back({(double)gidx + (k + 0.5) / sl.count, WaveWork{sl.t, (sl.first + k * sl.step) * G}});
      }
      ++gidx;
    }
    std::stable_sort(keyed.begin(), keyed.end(),
                     [](const std::pair<double, WaveWork>& p, const std::pair<double, WaveWork>& q) { return p.first < q.first; });
    for (auto& kv : keyed) list.push_back(kv.second);
    xcd_start[x + 1] = (int64_t)list.size();
    longest = std::max<int64_t>(longest, (int64_t)keyed.size());
  }
  out->num_waves = longest;
  HIP_TRY(hipMalloc((void**)&out->d_work, sizeof(WaveWork) * list.size()));
  HIP_TRY(hipMemcpy(out->d_work, list.data(), sizeof(WaveWork) * list.size(), hipMemcpyHostToDevice));
  HIP_TRY(hipMalloc((void**)&out->d_xcd_start, sizeof(int64_t) * 9));
  HIP_TRY(hipMemcpy(out->d_xcd_start, xcd_start.data(), sizeof(int64_t) * 9, hipMemcpyHostToDevice));
  return 0;
}

// Cached work lists beyond this many: the least recently used one that no graph can hold is dropped.
constexpr size_t MAX_CACHED_WORK = 16;

} // namespace

extern "C" {

int fbgemm_amd_tbe_plan_create(
    fbgemm_amd_tbe_plan** out, int32_t T, const int64_t* weights_offsets,
    const uint8_t* weights_tys, const int32_t* D_offsets, const int32_t* placements,
    int64_t dev_bytes, int64_t uvm_bytes, int64_t row_alignment) {
  if (!out || T <= 0 || !weights_offsets || !weights_tys || !D_offsets)
    return fail(FBGEMM_AMD_E_ARG, "bad plan arguments");
  if (row_alignment <= 0) row_alignment = 1;
  // owned here until it is handed out: every early return below frees the plan and what it holds
  std::unique_ptr<fbgemm_amd_tbe_plan, void (*)(fbgemm_amd_tbe_plan*)> owner(new fbgemm_amd_tbe_plan(), fbgemm_amd_tbe_plan_destroy);
  fbgemm_amd_tbe_plan* plan = owner.get();
  plan->T = T;
  plan->total_D = D_offsets[T];
  plan->row_alignment = row_alignment;
  plan->tables.resize(T);
  HIP_TRY(hipGetDevice(&plan->device));

  // Rows per table are inferred from the distance to the next distinct
  // offset in the same buffer, the last table being bounded by the buffer
  // (embedding_forward_quantized_cpu_template.cpp:330-341,372-380).
  std::vector<int64_t> phys[2];
  for (int t = 0; t < T; ++t) phys[(placements && placements[t] != 0) ? 1 : 0].push_back(weights_offsets[t]);
  for (auto& p : phys) {
    std::sort(p.begin(), p.end());
    p.erase(std::unique(p.begin(), p.end()), p.end());
  }
  for (int t = 0; t < T; ++t) {
    TableDesc& d = plan->tables[t];
    memset(&d, 0, sizeof(d));
    d.ty = weights_tys[t];
    if (type_bits(d.ty) == 0) {
      return fail(FBGEMM_AMD_E_UNSUPPORTED, "table %d: weight type %d is not supported", t, d.ty);
    }
    d.D = D_offsets[t + 1] - D_offsets[t];
    if (d.D <= 0) {
      return fail(FBGEMM_AMD_E_ARG, "table %d: D_offsets must increase", t);
    }
    d.out_col = D_offsets[t];
    d.placement = (placements && placements[t] != 0) ? 1 : 0;
    d.weights_offset = weights_offsets[t];
    d.row_stride = fbgemm_amd_padded_row_size_in_bytes(d.D, d.ty, (int32_t)row_alignment, 4);
    const auto& p = phys[d.placement];
    auto it = std::upper_bound(p.begin(), p.end(), d.weights_offset);
    const int64_t next = it != p.end() ? *it : (d.placement ? uvm_bytes : dev_bytes);
    d.num_rows = std::max<int64_t>(0, (next - d.weights_offset) / d.row_stride);
    d.skip_minus_one = 1;
    plan->has_fp8 = plan->has_fp8 || d.ty == ST_FP8;
    const bool q = quantised(d.ty);
    d.sb_fp32 = 0;
    d.sb_off = 0;
    d.data_off = q ? 4 : 0;
    // weights buffers come from hipMalloc / torch: at least 256-byte aligned
    plan_lanes(d, 0, plan->total_D, q, false);
    d.lanes_recip = (65536 + d.lanes - 1) / d.lanes;
    d.bags = bags_per_wave(d.lanes, d.packed);
  }
  HIP_TRY(hipMalloc((void**)&plan->d_D_offsets, sizeof(int32_t) * (T + 1)));
  HIP_TRY(hipMemcpy(plan->d_D_offsets, D_offsets, sizeof(int32_t) * (T + 1), hipMemcpyHostToDevice));
  for (int t = 0; t < T; ++t) plan->max_D = std::max(plan->max_D, D_offsets[t + 1] - D_offsets[t]);
  HIP_TRY(hipMalloc((void**)&plan->d_tables, sizeof(TableDesc) * T));
  HIP_TRY(hipMemcpy(plan->d_tables, plan->tables.data(), sizeof(TableDesc) * T, hipMemcpyHostToDevice));
  plan->tables_packed = plan->tables;
  bool any_packed = false;
  for (int t = 0; t < T; ++t) {
    TableDesc& d = plan->tables_packed[t];
    plan_lanes(d, 0, plan->total_D, quantised(d.ty), true);
    d.lanes_recip = (65536 + d.lanes - 1) / d.lanes;
    d.bags = bags_per_wave(d.lanes, d.packed);
    any_packed = any_packed || d.packed;
  }
  if (any_packed) {
    HIP_TRY(hipMalloc((void**)&plan->d_tables_packed, sizeof(TableDesc) * T));
    HIP_TRY(hipMemcpy(plan->d_tables_packed, plan->tables_packed.data(), sizeof(TableDesc) * T, hipMemcpyHostToDevice));
  } else {
    plan->tables_packed.clear();
  }
  plan->tables_narrow = plan->tables;
  for (int t = 0; t < T; ++t) {
    TableDesc& d = plan->tables_narrow[t];
    plan_lanes(d, 0, plan->total_D, quantised(d.ty), false, true);
    d.lanes_recip = (65536 + d.lanes - 1) / d.lanes;
    d.bags = bags_per_wave(d.lanes, d.packed);
  }
  HIP_TRY(hipMalloc((void**)&plan->d_tables_narrow, sizeof(TableDesc) * T));
  HIP_TRY(hipMemcpy(plan->d_tables_narrow, plan->tables_narrow.data(), sizeof(TableDesc) * T, hipMemcpyHostToDevice));
  *out = owner.release();
  return 0;
}

void fbgemm_amd_tbe_plan_destroy(fbgemm_amd_tbe_plan* plan) {
  if (!plan) return;
  (void)hipDeviceSynchronize();
  for (auto& kv : plan->work) free_work(kv.second);
  if (plan->d_tables) (void)hipFree(plan->d_tables);
  if (plan->d_tables_packed) (void)hipFree(plan->d_tables_packed);
  if (plan->d_tables_narrow) (void)hipFree(plan->d_tables_narrow);
  if (plan->d_D_offsets) (void)hipFree(plan->d_D_offsets);
  if (plan->pooled_tmp) (void)hipFree(plan->pooled_tmp);
  if (plan->seg_offsets) (void)hipFree(plan->seg_offsets);
  if (plan->seg_partial) (void)hipFree(plan->seg_partial);
  if (plan->shared_done) (void)hipEventDestroy(plan->shared_done);
  if (plan->d_rank_records) (void)hipFree(plan->d_rank_records);
  if (plan->d_rank_offsets) (void)hipFree(plan->d_rank_offsets);
  if (plan->d_rank_remap_offsets) (void)hipFree(plan->d_rank_remap_offsets);
  delete plan;
}

int fbgemm_amd_tbe_plan_set_fp8(fbgemm_amd_tbe_plan* plan, int32_t exponent_bits, int32_t exponent_bias) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  // embedding_forward_quantized_cpu_template.cpp (check_fp8_params): both must be given
  if (exponent_bits < 1 || exponent_bits > 6 || exponent_bias < 0 || exponent_bias > 253)
    return fail(FBGEMM_AMD_E_ARG, "fp8 needs 1..6 exponent bits and a bias in 0..253");
  std::lock_guard<std::mutex> lk(plan->mu);
  plan->fp8_shift = 16 + exponent_bits;
  const uint32_t mult_bits = (uint32_t)(127 + (127 - exponent_bias)) << 23; // 2^(127 - bias)
  memcpy(&plan->fp8_mult, &mult_bits, 4);
  return 0;
}

int64_t fbgemm_amd_tbe_plan_num_rows(const fbgemm_amd_tbe_plan* plan, int32_t t) {
  return (plan && t >= 0 && t < plan->T) ? plan->tables[t].num_rows : -1;
}
int64_t fbgemm_amd_tbe_plan_row_bytes(const fbgemm_amd_tbe_plan* plan, int32_t t) {
  return (plan && t >= 0 && t < plan->T) ? plan->tables[t].row_stride : -1;
}

int fbgemm_amd_tbe_forward(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t pooling_mode,
    const float* d_indice_weights, int32_t output_ty, void* d_output, void* d_status,
    void* stream_) {
  return fbgemm_amd_tbe_forward_pruned(plan, d_dev_weights, d_uvm_weights, d_indices, d_offsets, index_bits,
                                       indices_numel, offsets_numel, pooling_mode, d_indice_weights, output_ty,
                                       d_output, nullptr, 32, nullptr, 0, d_status, stream_);
}

} // extern "C"

namespace {
// A forward's use of the scratch all streams of a plan share (the float scratch of the 8-bit pooled
// output, the segment offsets and partial sums of split bags). begin(): from here to the end of
// the scope no other host thread enqueues such a forward of the plan, and if the last one ran on
// another stream this stream waits, on the device, for the event recorded behind it. The end of
// the scope records that event behind this forward. Under stream capture nothing is recorded or
// waited for (a graph cannot wait for work outside it): captured forwards of one plan that use
// this scratch are the caller's to order.
// Buffer k of a work set's bag orders, with the redo queue of the four-waves-per-SIMD lean
// instance when the set uses it. Allocates: not under stream capture.
int make_order_slot(fbgemm_amd_tbe_plan::Work& W, int k, int32_t T, int32_t B) {
  HIP_TRY(hipMalloc((void**)&W.d_order[k], sizeof(BagEntry) * (size_t)T * (size_t)B));
  if (W.lean_wide4 && W.lean.num_waves > 0) {
    HIP_TRY(hipMalloc((void**)&W.d_redo[k], sizeof(WaveWork) * (size_t)W.lean.num_waves));
    HIP_TRY(hipMalloc((void**)&W.d_redo_count[k], 2 * sizeof(int32_t)));
    const int32_t zeros[2] = {0, 0};
    HIP_TRY(hipMemcpy(W.d_redo_count[k], zeros, sizeof(zeros), hipMemcpyHostToDevice));
  }
  return 0;
}

struct SharedScratchUse {
  fbgemm_amd_tbe_plan* plan = nullptr;
  hipStream_t stream = nullptr;
  bool record = false;
  std::unique_lock<std::mutex> host;
  int begin(fbgemm_amd_tbe_plan* p, hipStream_t s) {
    if (plan) return 0; // already begun
    plan = p;
    stream = s;
    host = std::unique_lock<std::mutex>(p->shared_mu);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(s, &cap);
    if (cap != hipStreamCaptureStatusNone) return 0;
    if (!p->shared_done) HIP_TRY(hipEventCreateWithFlags(&p->shared_done, hipEventDisableTiming));
    if (p->shared_used && p->shared_stream != s) HIP_TRY(hipStreamWaitEvent(s, p->shared_done, 0));
    record = true;
    return 0;
  }
  ~SharedScratchUse() {
    if (!record) return;
    if (hipEventRecord(plan->shared_done, stream) == hipSuccess) {
      plan->shared_stream = stream;
      plan->shared_used = true;
    } else {
      (void)hipGetLastError();
    }
  }
};

// The forward behind fbgemm_amd_tbe_forward[_pruned]. offset_bits: the width of d_offsets (the
// operator's offsets have the width of its indices; the segment offsets of split bags are int64).
int tbe_forward_impl(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits, int32_t offset_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t pooling_mode,
    const float* d_indice_weights, int32_t output_ty, void* d_output,
    const void* d_index_remappings, int32_t remap_bits, const int64_t* d_index_remappings_offsets,
    int64_t index_remappings_offsets_numel, void* d_status, void* stream_, bool allow_split, uint8_t* d_q8_out = nullptr) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  if (d_index_remappings && (!d_index_remappings_offsets || (remap_bits != 32 && remap_bits != 64)))
    return fail(FBGEMM_AMD_E_ARG, "a remap array needs its T+1 offsets and 32- or 64-bit entries");
  // the kernels read offsets[t] and offsets[t + 1] for every t the plan has (one per FEATURE of the operator)
  if (d_index_remappings && index_remappings_offsets_numel != (int64_t)plan->T + 1)
    return fail(FBGEMM_AMD_E_ARG, "index_remappings_offsets holds %lld entries, the plan's %d tables need %d",
                (long long)index_remappings_offsets_numel, plan->T, plan->T + 1);
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  if (output_ty == ST_INT8) {
    // The reference's GPU operator quantizes every table's pooled vector row-wise to 8 bits in its
    // output stage ([B, total_D + 8 T]: D_t bytes, fp32 scale, fp32 bias per table;
    // embedding_forward_quantized_split_nbit_kernel_template.cu:535-566). Here: the lean kernel
    // does the same for its tables (lean_store_q8); the other tables, and forwards whose bags are
    // cut into segments, go as floats into plan-owned scratch, and one more launch quantizes
    // their (bag, table) segments.
    if (offsets_numel < 1 || (offsets_numel - 1) % plan->T != 0) return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
    const int64_t B = (offsets_numel - 1) / plan->T;
    if (B == 0) return 0;
    if (!d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
    return tbe_forward_impl(plan, d_dev_weights, d_uvm_weights, d_indices, d_offsets, index_bits, offset_bits,
                            indices_numel, offsets_numel, pooling_mode, d_indice_weights, ST_FP32, nullptr,
                            d_index_remappings, remap_bits, d_index_remappings_offsets,
                            index_remappings_offsets_numel, d_status, stream_, allow_split, (uint8_t*)d_output);
  }
  if (output_ty != ST_FP32 && output_ty != ST_FP16 && output_ty != ST_BF16)
    return fail(FBGEMM_AMD_E_UNSUPPORTED, "output type %d is not supported", output_ty);
  if (pooling_mode != FBGEMM_AMD_POOL_SUM && pooling_mode != FBGEMM_AMD_POOL_MEAN)
    return fail(FBGEMM_AMD_E_UNSUPPORTED, "pooling mode %d is not supported", pooling_mode);
  if (!d_status) return fail(FBGEMM_AMD_E_ARG, "d_status is null");
  if (offsets_numel < 1 || (offsets_numel - 1) % plan->T != 0)
    return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
  const int64_t B64 = (offsets_numel - 1) / plan->T;
  if (B64 == 0) return 0;
  if (B64 > 0x7fffffffLL) return fail(FBGEMM_AMD_E_ARG, "B exceeds 2^31-1");
  const int32_t B = (int32_t)B64;
  if (!d_offsets || (!d_output && !d_q8_out) || (indices_numel > 0 && !d_indices)) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  // the lane shapes of the plan assume what every device allocator gives (the
  // reference's kernels load uint4 from the same buffers)
  if ((uintptr_t)d_dev_weights % 16 || (uintptr_t)d_uvm_weights % 16)
    return fail(FBGEMM_AMD_E_ARG, "weights buffers must be 16-byte aligned");
  hipStream_t stream = (hipStream_t)stream_;
  SharedScratchUse shared; // begun where the forward turns out to use the plan's shared scratch
  // 8-bit pooled output: the float scratch [B, total_D] for what the lean kernel does not
  // quantize itself, made when a forward first needs it (not under a stream capture)
  auto pooled_scratch = [&](float** out) -> int {
    std::lock_guard<std::mutex> lk(plan->mu);
    const int64_t need = (int64_t)B * plan->total_D;
    if (plan->pooled_tmp_cap < need) {
      hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
      (void)hipStreamIsCapturing(stream, &cap);
      if (cap != hipStreamCaptureStatusNone)
        return fail(FBGEMM_AMD_E_ARG, "the first 8-bit forward of this size allocates float scratch: run it once outside the stream capture");
    }
    if (int rc = grow(&plan->pooled_tmp, &plan->pooled_tmp_cap, need, stream)) return rc;
    *out = plan->pooled_tmp;
    return 0;
  };
  if (plan->has_fp8 && plan->fp8_shift == 0)
    return fail(FBGEMM_AMD_E_ARG, "the plan holds FP8 tables: set their exponent bits and bias first (fbgemm_amd_tbe_plan_set_fp8)");

  // Few, long bags, and the plan accepts sums in another order: every bag is cut into K segments that
  // are pooled as bags of their own into fp32 partial sums, which a second launch adds up in order.
  // (Only when every table has rows the tolerance-grade arithmetic applies to: fp16 / fp32 / 2-bit
  // / odd-shaped tables are summed the reference's way in either mode, and a bag cut into
  // segments is not.)
  bool all_fast_rows = true;
  for (const TableDesc& d : plan->tables) all_fast_rows = all_fast_rows && (d.ty == ST_INT4 || d.ty == ST_INT8);
  if (allow_split && plan->accumulate == FBGEMM_AMD_ACC_FAST && all_fast_rows && (int64_t)B * 32 <= 0x7fffffffLL) {
    int64_t wide_waves = 0;
    for (const TableDesc& d : plan->tables) wide_waves += (B + d.bags - 1) / d.bags;
    const int K = split_factor(wide_waves, indices_numel / ((int64_t)plan->T * B));
    if (K > 1) {
      if (int rc = shared.begin(plan, stream)) return rc;
      hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
      (void)hipStreamIsCapturing(stream, &cap);
      const int64_t vbags = (int64_t)plan->T * B * K;
      int64_t* voff;
      float* partial;
      {
        std::lock_guard<std::mutex> lk(plan->mu);
        const bool fits = plan->seg_offsets_cap >= vbags + 1 && plan->seg_partial_cap >= (int64_t)B * K * plan->total_D;
        if (!fits && cap != hipStreamCaptureStatusNone)
          return fail(FBGEMM_AMD_E_ARG, "the first forward of this size allocates the scratch of split bags: run it once outside the stream capture");
        if (int rc = grow(&plan->seg_offsets, &plan->seg_offsets_cap, vbags + 1, stream)) return rc;
        if (int rc = grow(&plan->seg_partial, &plan->seg_partial_cap, (int64_t)B * K * plan->total_D, stream)) return rc;
        voff = plan->seg_offsets;
        partial = plan->seg_partial;
      }
      HIP_TRY(launch_split_offsets(d_offsets, offset_bits == 64, (int64_t)plan->T * B, K, false, indices_numel, voff, (Status*)d_status, stream));
      if (int rc = tbe_forward_impl(plan, d_dev_weights, d_uvm_weights, d_indices, voff, index_bits, 64, indices_numel, vbags + 1,
                                    FBGEMM_AMD_POOL_SUM, d_indice_weights, ST_FP32, partial, d_index_remappings, remap_bits,
                                    d_index_remappings_offsets, index_remappings_offsets_numel, d_status, stream_, false))
        return rc;
      if (d_q8_out) {
        float* tmp = nullptr;
        if (int rc = pooled_scratch(&tmp)) return rc;
        d_output = tmp;
      }
      HIP_TRY(launch_combine_segments(partial, plan->total_D, B, K, plan->T, plan->d_D_offsets, 0, d_offsets, offset_bits == 64,
                                      pooling_mode == FBGEMM_AMD_POOL_MEAN, d_output, output_ty, plan->total_D, stream));
      if (d_q8_out)
        HIP_TRY(launch_quantize_segments((const float*)d_output, B, plan->T, plan->d_D_offsets, (int32_t)plan->total_D, plan->max_D,
                                         d_q8_out, nullptr, 0, stream));
      return 0;
    }
  }

  // Bags laid end to end save a line request per row and cost about a fifth more
  // arithmetic on the tables they apply to. With short bags the per-bag work
  // makes the kernel arithmetic-bound and the saving does not pay (measured: 15
  // rows per bag loses 9 %, 30 rows per bag gains 5 %).
  static const int packed_mode = env_int("FBGEMM_AMD_PACKED", 1); // 0 never, 1 by bag length, 2 always
  // A forward of fewer than four waves per compute unit is bound by the chain of memory round
  // trips inside a wave: 4-byte lanes spread its bags over four times the waves.
  const bool lean = lean_enabled();
  fbgemm_amd_tbe_plan::Work w;
  int variant, order_slot = 0;
  // what the launches below take from the plan, read under its lock
  bool exact = true;
  const RankRecord* rank_records = nullptr;
  const int64_t* rank_offsets = nullptr;
  bool reuse_order = false;
  bool use_w4 = false;  // the lean tables take the four-waves-per-SIMD instance
  int measure_w4 = -1;  // >= 0: this forward times its lean kernel (0 / 1: which one) for the work set's choice
  {
    std::lock_guard<std::mutex> lk(plan->mu);
    // the lane shapes depend on B and (through the average bag length) on the number of indices:
    // remember the choice of the last forward with the same B and about the same indices
    const int64_t bucket = indices_numel >> 16;
    if (plan->shape_B == B && plan->shape_bucket == bucket && plan->shape_narrow == narrow_below_waves()) {
      variant = plan->shape_variant;
    } else {
      int64_t wide_waves = 0;
      for (const TableDesc& d : plan->tables) {
        const int G = bags_per_wave(d.lanes, d.packed);
        wide_waves += (B + G - 1) / G;
      }
      const bool use_narrow = wide_waves < narrow_below_waves();
      const bool use_packed = !use_narrow && !plan->tables_packed.empty() &&
          (packed_mode == 2 || (packed_mode == 1 && indices_numel >= 20 * (int64_t)plan->T * B));
      variant = use_narrow ? 2 : (use_packed ? 1 : 0);
      plan->shape_B = B;
      plan->shape_bucket = bucket;
      plan->shape_variant = variant;
      plan->shape_narrow = narrow_below_waves();
    }
    const std::vector<TableDesc>& tables = variant == 2 ? plan->tables_narrow : (variant == 1 ? plan->tables_packed : plan->tables);
    const fbgemm_amd_tbe_plan::WorkKey key{B, variant, lean ? 1 : 0};
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(stream, &cap);
    const bool capturing = cap != hipStreamCaptureStatusNone;
    auto it = plan->work.find(key);
    if (it == plan->work.end()) {
      if (capturing)
        return fail(FBGEMM_AMD_E_ARG, "the first forward of a plan with a new batch size allocates its work lists: "
                    "run it once outside the stream capture");
      std::vector<int> lean_members, general_members;
      for (int t = 0; t < plan->T; ++t) (lean && lean_shape(tables[t]) ? lean_members : general_members).push_back(t);
      fbgemm_amd_tbe_plan::Work nw;
      // what is allocated below goes back when a later step fails
      struct Undo {
        fbgemm_amd_tbe_plan::Work* w;
        ~Undo() { if (w) free_work(*w); }
      } undo{&nw};
      nw.lean_wide4 = !lean_members.empty();
      for (int t : lean_members) nw.lean_wide4 = nw.lean_wide4 && lean_wide4_shape(tables[(size_t)t]);
      if (nw.lean_wide4)
        for (int k = 0; k < 2; ++k) HIP_TRY(hipEventCreateWithFlags(&nw.w4_ev[k], hipEventDefault));
      if (int rc = build_work_list(tables, lean_members, B, &nw.lean)) return rc;
      if (int rc = build_work_list(tables, general_members, B, &nw.general)) return rc;
      if (!general_members.empty()) {
        const std::vector<int32_t> ids(general_members.begin(), general_members.end());
        HIP_TRY(hipMalloc((void**)&nw.d_general_tables, sizeof(int32_t) * ids.size()));
        HIP_TRY(hipMemcpy(nw.d_general_tables, ids.data(), sizeof(int32_t) * ids.size(), hipMemcpyHostToDevice));
        nw.n_general_tables = (int32_t)ids.size();
      }
      // the bag order: one buffer for this stream, one ahead for the next stream
      for (int k = 0; k < 2; ++k)
        if (int rc = make_order_slot(nw, k, plan->T, B)) return rc;
      nw.order_stream[0] = stream;
      nw.order_claimed[0] = true;
      // A caller whose batch size keeps changing would grow this cache without bound. Past
      // MAX_CACHED_WORK entries the least recently used one goes, after the launches that may
      // still read it are done. Entries a forward under stream capture has used are never
      // dropped here: a captured graph holds their device pointers (fbgemm_amd_tbe_plan_trim
      // drops those too, and says what that means for graphs).
      if (plan->work.size() >= MAX_CACHED_WORK) {
        auto victim = least_recently_used_not_held(
            plan->work, [](const fbgemm_amd_tbe_plan::Work& e) { return e.pinned; },
            [](const fbgemm_amd_tbe_plan::Work& e) { return e.last_use; });
        if (victim != plan->work.end()) {
          HIP_TRY(hipDeviceSynchronize());
          free_work(victim->second);
          plan->work.erase(victim);
        }
      }
      it = plan->work.emplace(key, nw).first;
      undo.w = nullptr; // the cache owns it now
    }
    it->second.pinned = it->second.pinned || capturing;
    it->second.last_use = ++plan->use_clock;
    // this stream's bag-order buffer: the one it has, else one nobody has claimed, else (outside
    // a capture) a new one; with all of that exhausted the first buffer is shared, and forwards
    // of this plan on the streams that share it must not overlap
    fbgemm_amd_tbe_plan::Work& W = it->second;
    constexpr int NS = fbgemm_amd_tbe_plan::ORDER_SLOTS;
    order_slot = -1;
    for (int k = 0; k < NS && order_slot < 0; ++k)
      if (W.order_claimed[k] && W.order_stream[k] == stream) order_slot = k;
    for (int k = 0; k < NS && order_slot < 0; ++k)
      if (!W.order_claimed[k] && W.d_order[k]) order_slot = k;
    for (int k = 0; k < NS && order_slot < 0 && !capturing; ++k)
      if (!W.d_order[k]) {
        if (int rc = make_order_slot(W, k, plan->T, B)) return rc;
        order_slot = k;
      }
    if (order_slot < 0) order_slot = 0;
    if (!W.order_claimed[order_slot]) {
      W.order_claimed[order_slot] = true;
      W.order_stream[order_slot] = stream;
      // keep one buffer ahead for the next stream, when that is possible now
      if (!capturing)
        for (int k = 0; k < NS; ++k)
          if (!W.d_order[k]) {
            if (int rc = make_order_slot(W, k, plan->T, B)) return rc;
            break;
          }
    }
    // the slot's side stream (default priority, like every stream here) and its two events
    if (!capturing && !W.side_stream[order_slot] && W.lean.num_waves > 0 && W.general.num_waves > 0) {
      hipStream_t s2 = nullptr;
      hipEvent_t e1 = nullptr, e2 = nullptr;
      if (hipStreamCreateWithFlags(&s2, hipStreamNonBlocking) == hipSuccess &&
          hipEventCreateWithFlags(&e1, hipEventDisableTiming) == hipSuccess &&
          hipEventCreateWithFlags(&e2, hipEventDisableTiming) == hipSuccess) {
        W.side_stream[order_slot] = s2;
        W.side_fork[order_slot] = e1;
        W.side_join[order_slot] = e2;
      } else { // the forward works without them
        if (e1) (void)hipEventDestroy(e1);
        if (e2) (void)hipEventDestroy(e2);
        if (s2) (void)hipStreamDestroy(s2);
        (void)hipGetLastError();
      }
    }
    // the lean kernel of this forward, where there is a choice
    if (W.lean_wide4 && !d_q8_out && W.d_redo[order_slot] && W.d_redo_count[order_slot] && sort_bags_default() &&
        indices_numel >= (int64_t)SORT_MIN_LOOKUPS) {
      const int mode = wide4_mode();
      if (mode == 2) {
        use_w4 = true;
      } else if (mode == 1 && W.w4_decided >= 0) {
        use_w4 = W.w4_decided == 1;
      } else if (mode == 1 && !capturing && W.w4_ev[0] && W.w4_ev[1] && !W.w4_busy) {
        measure_w4 = W.w4_seen[0] <= W.w4_seen[1] ? 0 : 1;
        W.w4_seen[measure_w4] += 1;
        W.w4_busy = true;
        use_w4 = measure_w4 == 1;
      }
    }
    w = W;
    exact = plan->accumulate != FBGEMM_AMD_ACC_FAST;
    if (d_index_remappings && plan->d_rank_records && plan->rank_source == d_index_remappings && plan->rank_bits == remap_bits) {
      rank_records = plan->d_rank_records;
      rank_offsets = plan->d_rank_offsets;
      d_index_remappings_offsets = plan->d_rank_remap_offsets;
    }
    reuse_order = plan->reuse_order;
  }

  // a forward that times its lean kernel: when it leaves it waits for the second event, adds the
  // sample to the set's statistics, decides when there are enough, and gives the turn back
  struct Measuring {
    fbgemm_amd_tbe_plan* plan;
    fbgemm_amd_tbe_plan::WorkKey key;
    hipEvent_t start, stop;
    int which;
    bool recorded = false;
    ~Measuring() {
      if (which < 0) return;
      float ms = 0.0f;
      const bool have = recorded && hipEventSynchronize(stop) == hipSuccess && hipEventElapsedTime(&ms, start, stop) == hipSuccess && ms > 0.0f;
      if (!have) (void)hipGetLastError();
      std::lock_guard<std::mutex> lk(plan->mu);
      auto it = plan->work.find(key);
      if (it == plan->work.end() || it->second.w4_ev[1] != stop) return; // the set has been dropped meanwhile
      fbgemm_amd_tbe_plan::Work& W = it->second;
      W.w4_busy = false;
      if (have && W.w4_seen[which] > 1) { // the first sample of each kernel is not kept
        W.w4_ms[which] += ms;
        W.w4_samples[which] += 1;
      }
      if (W.w4_decided < 0 && W.w4_samples[0] >= 3 && W.w4_samples[1] >= 3)
        W.w4_decided = W.w4_ms[1] / (float)W.w4_samples[1] < 0.99f * W.w4_ms[0] / (float)W.w4_samples[0] ? 1 : 0;
    }
  } measuring{plan, fbgemm_amd_tbe_plan::WorkKey{B, variant, lean ? 1 : 0}, w.w4_ev[0], w.w4_ev[1], measure_w4};
  if (d_q8_out && w.general.num_waves > 0) {
    if (int rc = shared.begin(plan, stream)) return rc;
    float* tmp = nullptr;
    if (int rc = pooled_scratch(&tmp)) return rc;
    d_output = tmp;
  }
  LookupArgs a;
  memset(&a, 0, sizeof(a));
  a.tables = variant == 2 ? plan->d_tables_narrow : (variant == 1 ? plan->d_tables_packed : plan->d_tables);
  a.weights[0] = (const uint8_t*)d_dev_weights;
  a.weights[1] = (const uint8_t*)d_uvm_weights;
  a.indices = d_indices;
  a.offsets = d_offsets;
  a.off64 = offset_bits == 64;
  a.sample_weights = d_indice_weights;
  a.remap = d_index_remappings;
  a.remap_offsets = d_index_remappings ? d_index_remappings_offsets : nullptr;
  a.remap64 = remap_bits == 64;
  a.rank_records = rank_records;
  a.rank_offsets = rank_offsets;
  a.out = d_output;
  a.out_stride = plan->total_D;
  a.index_size = indices_numel;
  a.B = B;
  a.T = plan->T;
  a.out_ty = output_ty;
  a.normalize = pooling_mode == FBGEMM_AMD_POOL_MEAN;
  a.check_total = 0;
  a.out_aligned = (uintptr_t)d_output % 16 == 0;
  a.status = (Status*)d_status;
  a.fp8_shift = plan->fp8_shift;
  a.fp8_mult = plan->fp8_mult;
  if (sort_bags_default() && indices_numel >= (int64_t)SORT_MIN_LOOKUPS) {
    if (!reuse_order) HIP_TRY(launch_bag_order(d_offsets, offset_bits == 64, B, plan->T, w.d_order[order_slot], stream));
    a.order = w.d_order[order_slot];
  }
  // Tables for both kernels, and a forward long enough not to notice two events (the size from
  // which the bags are ordered): the general kernel runs on the slot's side stream, beside the
  // lean one, forked off behind the scheduler and joined before the forward's stream goes on.
  static const int side_enabled = env_int("FBGEMM_AMD_SIDE_STREAM", 1);
  hipStream_t side = (side_enabled && w.lean.num_waves > 0 && w.general.num_waves > 0 && a.order) ? w.side_stream[order_slot] : nullptr;
  if (w.general.num_waves > 0) {
    a.work = w.general.d_work;
    a.xcd_start = w.general.d_xcd_start;
    a.num_waves = w.general.num_waves;
    if (side) {
      HIP_TRY(hipEventRecord(w.side_fork[order_slot], stream));
      HIP_TRY(hipStreamWaitEvent(side, w.side_fork[order_slot], 0));
      HIP_TRY(launch_lookup(a, index_bits == 64, side));
      HIP_TRY(hipEventRecord(w.side_join[order_slot], side));
    }
  }
  if (w.lean.num_waves > 0) {
    LookupArgs l = a;
    l.work = w.lean.d_work;
    l.xcd_start = w.lean.d_xcd_start;
    l.num_waves = w.lean.num_waves;
    if (d_q8_out) { // the 8-bit pooled output of these tables is made here
      l.out = d_q8_out;
      l.out_ty = ST_INT8;
      l.out_stride = (int64_t)plan->total_D + 8 * (int64_t)plan->T;
      l.out_aligned = (uintptr_t)d_q8_out % 16 == 0;
    }
    // the four-waves-per-SIMD instance: forwards that order their bags (large ones: its second,
    // usually idle launch does not show there), float output
    const bool wide4 = use_w4 && a.order;
    if (wide4) {
      l.redo = w.d_redo[order_slot];
      l.redo_count = w.d_redo_count[order_slot];
    }
    if (measure_w4 >= 0) (void)hipEventRecord(w.w4_ev[0], stream);
    const hipError_t launched = launch_lookup_lean(l, index_bits == 64, exact, wide4, stream);
    if (measure_w4 >= 0 && launched == hipSuccess && hipEventRecord(w.w4_ev[1], stream) == hipSuccess) measuring.recorded = true;
    HIP_TRY(launched);
  }
  if (w.general.num_waves > 0) {
    if (side) HIP_TRY(hipStreamWaitEvent(stream, w.side_join[order_slot], 0));
    else HIP_TRY(launch_lookup(a, index_bits == 64, stream));
    if (d_q8_out)
      HIP_TRY(launch_quantize_segments((const float*)d_output, B, plan->T, plan->d_D_offsets, (int32_t)plan->total_D, plan->max_D,
                                       d_q8_out, w.lean.num_waves > 0 ? w.d_general_tables : nullptr, w.n_general_tables, stream));
  }
  return 0;
}
} // namespace

extern "C" {

int fbgemm_amd_tbe_forward_pruned(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t pooling_mode,
    const float* d_indice_weights, int32_t output_ty, void* d_output,
    const void* d_index_remappings, int32_t remap_bits, const int64_t* d_index_remappings_offsets,
    int64_t index_remappings_offsets_numel, void* d_status, void* stream) {
  return tbe_forward_impl(plan, d_dev_weights, d_uvm_weights, d_indices, d_offsets, index_bits, index_bits, indices_numel,
                          offsets_numel, pooling_mode, d_indice_weights, output_ty, d_output, d_index_remappings, remap_bits,
                          d_index_remappings_offsets, index_remappings_offsets_numel, d_status, stream, true);
}

int fbgemm_amd_tbe_plan_set_accumulate(fbgemm_amd_tbe_plan* plan, int32_t mode) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  if (mode != FBGEMM_AMD_ACC_EXACT && mode != FBGEMM_AMD_ACC_FAST)
    return fail(FBGEMM_AMD_E_ARG, "accumulate must be FBGEMM_AMD_ACC_EXACT or FBGEMM_AMD_ACC_FAST");
  std::lock_guard<std::mutex> lk(plan->mu);
  plan->accumulate = mode;
  return 0;
}

int fbgemm_amd_tbe_plan_set_index_remappings(
    fbgemm_amd_tbe_plan* plan, const void* d_index_remappings, int32_t remap_bits,
    const int64_t* index_remappings_offsets, int64_t index_remappings_offsets_numel, void* stream_) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> lk(plan->mu);
  // forget what was made from an earlier array (after the forwards that may still read it)
  if (plan->d_rank_records || plan->d_rank_offsets || plan->d_rank_remap_offsets) {
    HIP_TRY(hipDeviceSynchronize());
    if (plan->d_rank_records) (void)hipFree(plan->d_rank_records);
    if (plan->d_rank_offsets) (void)hipFree(plan->d_rank_offsets);
    if (plan->d_rank_remap_offsets) (void)hipFree(plan->d_rank_remap_offsets);
    plan->d_rank_records = nullptr;
    plan->d_rank_offsets = nullptr;
    plan->d_rank_remap_offsets = nullptr;
  }
  plan->rank_source = nullptr;
  plan->rank_tables = 0;
  if (!d_index_remappings) return 0;
  if (remap_bits != 32 && remap_bits != 64) return fail(FBGEMM_AMD_E_ARG, "remap entries are 32 or 64 bits wide");
  if (!index_remappings_offsets || index_remappings_offsets_numel != (int64_t)plan->T + 1)
    return fail(FBGEMM_AMD_E_ARG, "index_remappings_offsets must hold T+1 = %d entries (on the host)", plan->T + 1);
  const int T = plan->T;
  std::vector<int64_t> first(T, -1);
  int64_t words = 0, max_partials = 1;
  for (int t = 0; t < T; ++t) {
    const int64_t rows = index_remappings_offsets[t + 1] - index_remappings_offsets[t];
    if (rows < 0) return fail(FBGEMM_AMD_E_ARG, "index_remappings_offsets must not decrease");
    if (rows == 0) continue;
    first[t] = words;
    words += remap_rank_words(rows);
    max_partials = std::max(max_partials, remap_rank_partials(rows));
  }
  if (words == 0) return 0;
  RankRecord* records = nullptr;
  int64_t* partial = nullptr;
  int32_t* flags = nullptr;
  auto drop = [&]() {
    if (records) (void)hipFree(records);
    if (partial) (void)hipFree(partial);
    if (flags) (void)hipFree(flags);
  };
#define HIP_TRY_DROP(expr)                                                              \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess) {                                                             \
      drop();                                                                           \
      return fail(FBGEMM_AMD_E_HIP, "%s: %s", #expr, hipGetErrorString(e_));            \
    }                                                                                   \
  } while (0)
  HIP_TRY_DROP(hipMalloc((void**)&records, sizeof(RankRecord) * (size_t)words));
  HIP_TRY_DROP(hipMalloc((void**)&partial, sizeof(int64_t) * (size_t)max_partials));
  HIP_TRY_DROP(hipMalloc((void**)&flags, sizeof(int32_t) * (size_t)T));
  HIP_TRY_DROP(hipMemsetAsync(flags, 0, sizeof(int32_t) * (size_t)T, stream));
  const size_t esz = remap_bits / 8;
  for (int t = 0; t < T; ++t) {
    if (first[t] < 0) continue;
    const int64_t rows = index_remappings_offsets[t + 1] - index_remappings_offsets[t];
    HIP_TRY_DROP(launch_remap_rank_build((const char*)d_index_remappings + (size_t)index_remappings_offsets[t] * esz,
                                         remap_bits == 64, rows, records + first[t], partial, flags + t, stream));
  }
  std::vector<int32_t> h_flags(T, 0);
  HIP_TRY_DROP(hipMemcpyAsync(h_flags.data(), flags, sizeof(int32_t) * (size_t)T, hipMemcpyDeviceToHost, stream));
  HIP_TRY_DROP(hipStreamSynchronize(stream));
  int used = 0;
  for (int t = 0; t < T; ++t) {
    if (first[t] >= 0 && h_flags[t] != 0) first[t] = -1; // not order-preserving: the forward reads the array
    used += first[t] >= 0;
  }
  int64_t* d_first = nullptr;
  int64_t* d_offs = nullptr;
  if (used > 0) {
    hipError_t e = hipMalloc((void**)&d_first, sizeof(int64_t) * (size_t)T);
    if (e == hipSuccess) e = hipMemcpy(d_first, first.data(), sizeof(int64_t) * (size_t)T, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&d_offs, sizeof(int64_t) * (size_t)(T + 1));
    if (e == hipSuccess) e = hipMemcpy(d_offs, index_remappings_offsets, sizeof(int64_t) * (size_t)(T + 1), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      if (d_first) (void)hipFree(d_first);
      if (d_offs) (void)hipFree(d_offs);
      drop();
      return fail(FBGEMM_AMD_E_HIP, "rank offsets: %s", hipGetErrorString(e));
    }
    plan->d_rank_records = records;
    records = nullptr;
    plan->d_rank_offsets = d_first;
    plan->d_rank_remap_offsets = d_offs;
    plan->rank_source = d_index_remappings;
    plan->rank_bits = remap_bits;
    plan->rank_tables = used;
  }
  drop();
#undef HIP_TRY_DROP
  return 0;
}

int32_t fbgemm_amd_tbe_plan_rank_tables(const fbgemm_amd_tbe_plan* plan) { return plan ? plan->rank_tables : -1; }

int fbgemm_amd_tbe_plan_trim(fbgemm_amd_tbe_plan* plan) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  std::lock_guard<std::mutex> lk(plan->mu);
  HIP_TRY(hipDeviceSynchronize());
  for (auto& kv : plan->work) free_work(kv.second);
  plan->work.clear();
  return 0;
}

int64_t fbgemm_amd_tbe_plan_cached_work(const fbgemm_amd_tbe_plan* plan) {
  return plan ? (int64_t)plan->work.size() : -1;
}

int64_t fbgemm_amd_tbe_plan_pinned_work(fbgemm_amd_tbe_plan* plan) {
  if (!plan) return -1;
  std::lock_guard<std::mutex> lk(plan->mu);
  int64_t n = 0;
  for (const auto& kv : plan->work) n += kv.second.pinned ? 1 : 0;
  return n;
}

int fbgemm_amd_tbe_forward_nobag(
    fbgemm_amd_tbe_plan* plan, const void* d_dev_weights, const void* d_uvm_weights,
    const void* d_indices, const void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t D, int32_t output_ty,
    void* d_output, void* d_status, void* stream) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  const bool copy_rows = output_ty == ST_INT8 || output_ty == ST_INT4;
  if (!copy_rows && output_ty != ST_FP32 && output_ty != ST_FP16 && output_ty != ST_BF16)
    return fail(FBGEMM_AMD_E_UNSUPPORTED, "output type %d is not supported", output_ty);
  if (!d_status) return fail(FBGEMM_AMD_E_ARG, "d_status is null");
  if (D <= 0) return fail(FBGEMM_AMD_E_ARG, "D must be positive");
  if (offsets_numel < 1 || (offsets_numel - 1) % plan->T != 0)
    return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
  const int64_t B64 = (offsets_numel - 1) / plan->T;
  if (B64 > 0x7fffffffLL) return fail(FBGEMM_AMD_E_ARG, "B exceeds 2^31-1");
  if (B64 == 0 || indices_numel == 0) return 0;
  if (!d_offsets || !d_output || !d_indices) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  if (plan->has_fp8 && plan->fp8_shift == 0)
    return fail(FBGEMM_AMD_E_ARG, "the plan holds FP8 tables: set their exponent bits and bias first (fbgemm_amd_tbe_plan_set_fp8)");
  for (int t = 0; t < plan->T; ++t) {
    const TableDesc& d = plan->tables[t];
    if (d.D != D) return fail(FBGEMM_AMD_E_ARG, "table %d has D = %d: without pooling all tables share D = %d", t, d.D, D);
    // embedding_forward_quantized_cpu_template.cpp:357-359
    if (copy_rows && d.ty != output_ty)
      return fail(FBGEMM_AMD_E_ARG, "table %d: int8 / int4 output copies rows and needs weights of the same type", t);
    const int eb = type_bits(d.ty) / 8;
    if (eb > 1 && (d.weights_offset % eb || d.row_stride % eb))
      return fail(FBGEMM_AMD_E_ARG, "table %d: rows are not aligned to their elements", t);
  }
  HIP_TRY(launch_sequence_lookup(plan->d_tables, (const uint8_t*)d_dev_weights, (const uint8_t*)d_uvm_weights, d_indices,
                                 index_bits == 64, d_offsets, (int32_t)B64, plan->T, indices_numel, D, output_ty,
                                 d_output, plan->fp8_shift, plan->fp8_mult, (Status*)d_status, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_tbe_plan_reuse_order(fbgemm_amd_tbe_plan* plan, int32_t on) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  std::lock_guard<std::mutex> lk(plan->mu);
  plan->reuse_order = on != 0;
  return 0;
}

namespace {
int check_quant_format(int32_t bit_rate, int32_t sb_float, int32_t layout, int32_t cols, int64_t row_stride) {
  if (bit_rate != 2 && bit_rate != 4 && bit_rate != 8) return fail(FBGEMM_AMD_E_ARG, "bit_rate must be 2, 4 or 8");
  if (sb_float && bit_rate != 8) return fail(FBGEMM_AMD_E_ARG, "fp32 scale/bias go with 8-bit rows only");
  if (layout != FBGEMM_AMD_QLAYOUT_TRAILER && layout != FBGEMM_AMD_QLAYOUT_TBE) return fail(FBGEMM_AMD_E_ARG, "unknown row layout");
  if (cols <= 0) return fail(FBGEMM_AMD_E_ARG, "cols must be positive");
  const int epb = 8 / bit_rate;
  const int64_t need = (cols + epb - 1) / epb + ((sb_float && layout == FBGEMM_AMD_QLAYOUT_TRAILER) ? 8 : 4);
  if (row_stride < need) return fail(FBGEMM_AMD_E_ARG, "row stride %lld is below the %lld bytes a row takes", (long long)row_stride, (long long)need);
  return 0;
}
} // namespace

int fbgemm_amd_quantize_rowwise_min_max(
    const void* d_input, int32_t input_ty, int64_t rows, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int64_t out_row_stride, void* d_output, const void* d_rowwise_min_max, void* stream) {
  if (input_ty != ST_FP32 && input_ty != ST_FP16) return fail(FBGEMM_AMD_E_ARG, "input must be fp32 or fp16");
  if (rows < 0) return fail(FBGEMM_AMD_E_ARG, "rows must not be negative");
  if (int rc = check_quant_format(bit_rate, sb_float, layout, cols, out_row_stride)) return rc;
  if (rows == 0) return 0;
  if (!d_input || !d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_quantize_rowwise(d_input, input_ty == ST_FP16, rows, cols, bit_rate, sb_float, layout, out_row_stride,
                                  d_output, d_rowwise_min_max, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_quantize_rowwise(
    const void* d_input, int32_t input_ty, int64_t rows, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int64_t out_row_stride, void* d_output, void* stream) {
  return fbgemm_amd_quantize_rowwise_min_max(d_input, input_ty, rows, cols, bit_rate, sb_float, layout, out_row_stride,
                                             d_output, nullptr, stream);
}

int fbgemm_amd_dequantize_rowwise(
    const void* d_input, int64_t rows, int64_t in_row_stride, int32_t cols, int32_t bit_rate, int32_t sb_float,
    int32_t layout, int32_t output_ty, void* d_output, void* stream) {
  if (output_ty != ST_FP32 && output_ty != ST_FP16 && output_ty != ST_BF16) return fail(FBGEMM_AMD_E_ARG, "output must be fp32, fp16 or bf16");
  if (rows < 0) return fail(FBGEMM_AMD_E_ARG, "rows must not be negative");
  if (layout == FBGEMM_AMD_QLAYOUT_TBE && sb_float) return fail(FBGEMM_AMD_E_ARG, "TBE rows carry an fp16 scale/bias pair");
  if (int rc = check_quant_format(bit_rate, sb_float, layout, cols, in_row_stride)) return rc;
  if (rows == 0) return 0;
  if (!d_input || !d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_dequantize_rowwise(d_input, rows, in_row_stride, cols, bit_rate, sb_float, layout, output_ty, d_output,
                                    (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_float_to_hfp8(const float* d_input, int64_t n, int32_t ebits, int32_t exponent_bias, float max_pos,
                             uint8_t* d_output, void* stream) {
  if (n < 0) return fail(FBGEMM_AMD_E_ARG, "n must not be negative");
  if (ebits < 1 || ebits > 6 || exponent_bias < 0 || exponent_bias > 126) return fail(FBGEMM_AMD_E_ARG, "hfp8 needs 1..6 exponent bits and a bias in 0..126");
  if (!(max_pos > 0.0f)) return fail(FBGEMM_AMD_E_ARG, "max_pos must be positive");
  if (n == 0) return 0;
  if (!d_input || !d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_float_to_hfp8(d_input, n, ebits, exponent_bias, max_pos, d_output, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_hfp8_to_float(const uint8_t* d_input, int64_t n, int32_t ebits, int32_t exponent_bias, float* d_output,
                             void* stream) {
  if (n < 0) return fail(FBGEMM_AMD_E_ARG, "n must not be negative");
  if (ebits < 1 || ebits > 6 || exponent_bias < 0 || exponent_bias > 253) return fail(FBGEMM_AMD_E_ARG, "hfp8 needs 1..6 exponent bits and a bias in 0..253");
  if (n == 0) return 0;
  if (!d_input || !d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_hfp8_to_float(d_input, n, ebits, exponent_bias, d_output, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_rowwise_prune_map(const float* d_indicator, int64_t rows, double threshold, int32_t use_abs,
                                 int64_t min_non_pruned_rows, int32_t index_bits, void* d_remap, int64_t* num_kept,
                                 void* stream_) {
  if (rows < 0) return fail(FBGEMM_AMD_E_ARG, "rows must not be negative");
  if (!(threshold >= 0.0)) return fail(FBGEMM_AMD_E_ARG, "Threshold should be greater than or equal to zero.");
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  if (index_bits == 32 && rows > 0x7fffffffLL) return fail(FBGEMM_AMD_E_ARG, "rows do not fit 32-bit ids");
  if (!num_kept) return fail(FBGEMM_AMD_E_ARG, "num_kept is null");
  *num_kept = 0;
  if (rows == 0) return 0;
  if (!d_indicator || !d_remap) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> lk(g_mu);
  DeviceScratch* s;
  if (int rc = get_scratch(&s)) return rc;
  // the block sums, and one more slot for the count that comes back
  const int64_t np = prune_partials(rows);
  if (int rc = grow(&s->partial, &s->partial_cap, np + 1, stream)) return rc;
  HIP_TRY(launch_prune_map(d_indicator, rows, threshold, use_abs, min_non_pruned_rows, index_bits == 64, d_remap,
                           s->partial + np, s->partial, stream));
  HIP_TRY(hipMemcpyAsync(num_kept, s->partial + np, sizeof(int64_t), hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipStreamSynchronize(stream));
  return 0;
}

int fbgemm_amd_rowwise_prune_gather(const void* d_weights, int64_t rows, int64_t row_bytes, const void* d_remap,
                                    int32_t index_bits, void* d_output, int64_t output_rows, void* stream) {
  if (rows < 0 || row_bytes < 0 || output_rows < 0) return fail(FBGEMM_AMD_E_ARG, "negative size");
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  if (rows == 0 || row_bytes == 0 || output_rows == 0) return 0;
  if (!d_weights || !d_remap || !d_output) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_prune_gather(d_weights, rows, row_bytes, d_remap, index_bits == 64, d_output, output_rows, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_compressed_indices_remap(
    int32_t offsets_numel, const void* d_indices, int32_t index_bits, const int32_t* d_mapping, int64_t mapping_numel,
    const void* d_offsets, const float* d_weights, void* d_out_indices, void* d_out_offsets, float* d_out_weights,
    void* d_status, void* stream_) {
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  if (offsets_numel < 1) return fail(FBGEMM_AMD_E_ARG, "offsets must hold at least one entry");
  if (!d_offsets || !d_out_offsets || !d_mapping) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  if (mapping_numel < 0) return fail(FBGEMM_AMD_E_ARG, "mapping_numel must not be negative");
  hipStream_t stream = (hipStream_t)stream_;
  // the positions the reference walks: offsets[0] .. offsets[last] - 1
  const size_t eb = index_bits / 8;
  int64_t ends[2] = {0, 0};
  HIP_TRY(hipMemcpyAsync(&ends[0], d_offsets, eb, hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipMemcpyAsync(&ends[1], (const char*)d_offsets + (size_t)(offsets_numel - 1) * eb, eb, hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipStreamSynchronize(stream));
  if (index_bits == 32) {
    ends[0] = (int32_t)ends[0];
    ends[1] = (int32_t)ends[1];
  }
  const int64_t first = ends[0];
  const int64_t n = ends[1] > first ? ends[1] - first : 0;
  if (first < 0) return fail(FBGEMM_AMD_E_ARG, "offsets[0] is negative");
  if (n > 0 && (!d_indices || !d_out_indices)) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  if (n > 0 && d_weights && !d_out_weights) return fail(FBGEMM_AMD_E_ARG, "weights need out_weights");
  std::lock_guard<std::mutex> lk(g_mu);
  DeviceScratch* s;
  if (int rc = get_scratch(&s)) return rc;
  // one scratch buffer: n + 1 running counts (int64), then the n mapped rows (int32)
  if (int rc = grow(&s->fixed, &s->fixed_cap, (n + 1) + (n + 1) / 2 + 1, stream)) return rc;
  if (int rc = grow(&s->partial, &s->partial_cap, prune_partials(n + 1), stream)) return rc;
  HIP_TRY(launch_compressed_indices_remap(d_indices, index_bits == 64, d_mapping, mapping_numel, d_offsets, offsets_numel,
                                          d_weights, first, n, d_out_indices, d_out_offsets, d_out_weights, s->fixed,
                                          s->partial, reinterpret_cast<int32_t*>(s->fixed + n + 1),
                                          d_status ? (Status*)d_status : s->status, stream));
  return 0;
}

int fbgemm_amd_bounds_check_indices(
    const int64_t* d_rows_per_table, int32_t T, void* d_indices, void* d_offsets, int32_t index_bits,
    int64_t indices_numel, int64_t offsets_numel, int32_t bounds_check_mode, int64_t* d_warning,
    const int32_t* d_B_offsets, void* d_status, void* stream_) {
  if (T <= 0 || !d_rows_per_table) return fail(FBGEMM_AMD_E_ARG, "rows_per_table must hold T >= 1 entries");
  if (index_bits != 32 && index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "index_bits must be 32 or 64");
  if (bounds_check_mode < 0 || bounds_check_mode > 2) return fail(FBGEMM_AMD_E_ARG, "bounds_check_mode must be 0 (FATAL), 1 (WARNING) or 2 (IGNORE)");
  if (offsets_numel < 1 || !d_offsets) return fail(FBGEMM_AMD_E_ARG, "offsets must hold at least one entry");
  const int64_t total_B = offsets_numel - 1;
  // embedding_bounds_check_host_cpu.cpp:126-131
  if (!d_B_offsets && total_B % T != 0)
    return fail(FBGEMM_AMD_E_ARG, "offsets size %lld is not equal to B (%lld) * T (%d) + 1", (long long)offsets_numel,
                (long long)(total_B / T), T);
  if (indices_numel > 0 && !d_indices) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  if (bounds_check_mode == 1 && !d_warning) return fail(FBGEMM_AMD_E_ARG, "WARNING mode needs the warning counter");
  if (bounds_check_mode == 0 && !d_status) return fail(FBGEMM_AMD_E_ARG, "FATAL mode reports through d_status");
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> lk(g_mu);
  DeviceScratch* s;
  if (int rc = get_scratch(&s)) return rc;
  if (int rc = grow(&s->fixed, &s->fixed_cap, total_B + 1, stream)) return rc;
  if (int rc = grow(&s->partial, &s->partial_cap, bounds_check_partials(total_B), stream)) return rc;
  HIP_TRY(launch_bounds_check(d_rows_per_table, T, d_indices, d_offsets, index_bits == 64, indices_numel, total_B,
                              d_B_offsets ? 0 : total_B / T, d_B_offsets, bounds_check_mode, d_warning, s->fixed,
                              s->partial, (Status*)d_status, stream));
  return 0;
}

namespace {
inline uint64_t host_pruned_hash(uint64_t k, bool wide) {
  if (wide) { // MurmurHash3's 64-bit finalizer
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdull;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ull;
    k ^= k >> 33;
    return k;
  }
  uint32_t h = (uint32_t)k; // and its 32-bit one
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}
inline int64_t host_read(const void* p, bool wide, int64_t i) {
  return wide ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}
inline void host_write(void* p, bool wide, int64_t i, int64_t v) {
  if (wide) ((int64_t*)p)[i] = v;
  else ((int32_t*)p)[i] = (int32_t)v;
}
} // namespace

int fbgemm_amd_pruned_hashmap_insert_host(
    const void* h_indices, const void* h_dense_indices, const void* h_offsets, int32_t index_bits,
    int64_t offsets_numel, void* h_hash_table, int32_t hash_bits, const int64_t* h_hash_table_offsets, int32_t T) {
  if (T <= 0 || offsets_numel < 1 || (offsets_numel - 1) % T != 0) return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
  if ((index_bits != 32 && index_bits != 64) || (hash_bits != 32 && hash_bits != 64))
    return fail(FBGEMM_AMD_E_ARG, "index_bits/hash_bits must be 32 or 64");
  const int64_t B = (offsets_numel - 1) / T;
  if (B <= 0) return fail(FBGEMM_AMD_E_ARG, "pruned_hashmap_insert needs B > 0");
  if (!h_offsets || !h_hash_table_offsets) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  // a map without slots (no table is pruned) has nothing to insert into: the reference's loop skips such tables
  if (h_hash_table_offsets[T] - h_hash_table_offsets[0] <= 0) return 0;
  if (!h_indices || !h_dense_indices || !h_hash_table) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  const bool iw = index_bits == 64, hw = hash_bits == 64;
  for (int32_t t = 0; t < T; ++t) {
    const int64_t table_start = h_hash_table_offsets[t];
    const int64_t capacity = h_hash_table_offsets[t + 1] - table_start;
    if (capacity <= 0) continue;
    const int64_t lo = host_read(h_offsets, iw, (int64_t)t * B), hi = host_read(h_offsets, iw, (int64_t)(t + 1) * B);
    for (int64_t i = lo; i < hi; ++i) {
      const int64_t idx = host_read(h_indices, iw, i);
      const int64_t dense = host_read(h_dense_indices, iw, i);
      if (dense == -1) continue; // a pruned row is not in the map
      // the hash is taken of the id at the index width, as the reference takes it
      int64_t slot = (int64_t)(host_pruned_hash(iw ? (uint64_t)idx : (uint64_t)(uint32_t)idx, iw) % (uint64_t)capacity);
      int64_t probes = 0;
      for (;; ++probes) {
        if (probes == capacity) return fail(FBGEMM_AMD_E_ARG, "hash table of table %d is full", t);
        const int64_t key = host_read(h_hash_table, hw, 2 * (table_start + slot));
        if (key == -1 || key == idx) {
          host_write(h_hash_table, hw, 2 * (table_start + slot), idx);
          host_write(h_hash_table, hw, 2 * (table_start + slot) + 1, dense);
          break;
        }
        slot = slot + 1 == capacity ? 0 : slot + 1;
      }
    }
  }
  return 0;
}

int fbgemm_amd_pruned_hashmap_lookup(
    const void* d_indices, const void* d_offsets, int32_t index_bits, int64_t offsets_numel,
    const void* d_hash_table, int32_t hash_bits, const int64_t* d_hash_table_offsets, int32_t T,
    void* d_dense, void* stream) {
  if (T <= 0 || offsets_numel < 1 || (offsets_numel - 1) % T != 0) return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
  if ((index_bits != 32 && index_bits != 64) || (hash_bits != 32 && hash_bits != 64))
    return fail(FBGEMM_AMD_E_ARG, "index_bits/hash_bits must be 32 or 64");
  const int64_t B = (offsets_numel - 1) / T;
  if (B == 0) return 0;
  if (!d_indices || !d_offsets || !d_hash_table_offsets || !d_dense) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_pruned_hashmap_lookup(d_indices, d_offsets, index_bits == 64, d_hash_table, hash_bits == 64,
                                       d_hash_table_offsets, (int32_t)B, T, d_dense, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_pruned_array_lookup(
    const void* d_indices, const void* d_offsets, int32_t index_bits, int64_t offsets_numel,
    const void* d_remap, int32_t remap_bits, const int64_t* d_remap_offsets, int32_t T,
    void* d_dense, void* stream) {
  if (T <= 0 || offsets_numel < 1 || (offsets_numel - 1) % T != 0) return fail(FBGEMM_AMD_E_ARG, "offsets must hold T*B+1 entries");
  if ((index_bits != 32 && index_bits != 64) || (remap_bits != 32 && remap_bits != 64))
    return fail(FBGEMM_AMD_E_ARG, "index_bits/remap_bits must be 32 or 64");
  const int64_t B = (offsets_numel - 1) / T;
  if (B == 0) return 0;
  if (!d_indices || !d_offsets || !d_remap_offsets || !d_dense) return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_pruned_array_lookup(d_indices, d_offsets, index_bits == 64, d_remap, remap_bits == 64,
                                     d_remap_offsets, (int32_t)B, T, d_dense, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_tbe_inplace_update(
    fbgemm_amd_tbe_plan* plan, void* d_dev_weights, void* d_uvm_weights, const void* d_update_weights,
    int64_t update_weights_bytes, const int32_t* d_update_table_idx, const void* d_update_row_idx,
    int32_t row_index_bits, const int64_t* d_update_offsets, int64_t n, void* d_status, void* stream) {
  if (!plan) return fail(FBGEMM_AMD_E_ARG, "plan is null");
  if (row_index_bits != 32 && row_index_bits != 64) return fail(FBGEMM_AMD_E_ARG, "row_index_bits must be 32 or 64");
  if (n < 0 || update_weights_bytes < 0) return fail(FBGEMM_AMD_E_ARG, "negative size");
  if (n == 0) return 0;
  if (!d_update_weights || !d_update_table_idx || !d_update_row_idx || !d_update_offsets)
    return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  int64_t max_row_bytes = 0;
  for (int t = 0; t < plan->T; ++t) {
    const TableDesc& d = plan->tables[t];
    if (d.num_rows > 0 && !(d.placement ? d_uvm_weights : d_dev_weights))
      return fail(FBGEMM_AMD_E_ARG, "table %d lives in a weights buffer that was not passed", t);
    max_row_bytes = std::max(max_row_bytes, d.row_stride);
  }
  HIP_TRY(launch_inplace_update(plan->d_tables, plan->T, (uint8_t*)d_dev_weights, (uint8_t*)d_uvm_weights,
                                (const uint8_t*)d_update_weights, update_weights_bytes, d_update_table_idx,
                                d_update_row_idx, row_index_bits == 64, d_update_offsets, n, max_row_bytes,
                                (Status*)d_status, (hipStream_t)stream));
  return 0;
}

int fbgemm_amd_pruned_array_lookup_from_row_idx(
    const void* d_update_row_idx, int32_t index_bits, const int32_t* d_update_table_idx, int64_t n, const void* d_remap,
    int32_t remap_bits, const int64_t* d_remap_offsets, int32_t T, void* d_dense, void* stream) {
  if (T <= 0 || n < 0) return fail(FBGEMM_AMD_E_ARG, "bad sizes");
  if ((index_bits != 32 && index_bits != 64) || (remap_bits != 32 && remap_bits != 64))
    return fail(FBGEMM_AMD_E_ARG, "index_bits/remap_bits must be 32 or 64");
  if (n == 0) return 0;
  if (!d_update_row_idx || !d_update_table_idx || !d_remap_offsets || !d_dense)
    return fail(FBGEMM_AMD_E_ARG, "null data pointer");
  HIP_TRY(launch_remap_row_idx(d_update_row_idx, index_bits == 64, d_update_table_idx, d_remap, remap_bits == 64,
                               d_remap_offsets, T, n, d_dense, (hipStream_t)stream));
  return 0;
}

} // extern "C"
