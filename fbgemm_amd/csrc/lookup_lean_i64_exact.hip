// One instance of the lean pooled-lookup kernel.
#include "lookup_lean.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LEAN_LAUNCH(launch_lookup_lean_i64_exact, int64_t, true, false)
} // namespace fbgemm_amd
