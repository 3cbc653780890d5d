// One instance of the lean pooled-lookup kernel: 4-bit rows in bags of 8 lanes and more, four waves per SIMD.
#include "lookup_lean.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LEAN_WIDE4_LAUNCH(launch_lookup_lean_i64_exact_w4, int64_t, true)
} // namespace fbgemm_amd
