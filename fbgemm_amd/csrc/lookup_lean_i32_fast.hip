// One instance of the lean pooled-lookup kernel.
#include "lookup_lean.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LEAN_LAUNCH(launch_lookup_lean_i32_fast, int32_t, false, false)
} // namespace fbgemm_amd
