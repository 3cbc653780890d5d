// One instance of the lean pooled-lookup kernel: 4-bit rows in bags of 8 lanes and more, four waves per SIMD.
#include "lookup_lean.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LEAN_WIDE4_LAUNCH(launch_lookup_lean_i32_fast_w4, int32_t, false)
} // namespace fbgemm_amd
