// One instance of the lean pooled-lookup kernel: the one that writes the 8-bit pooled output.
#include "lookup_lean.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LEAN_LAUNCH(launch_lookup_lean_i64_exact_q8, int64_t, true, true)
} // namespace fbgemm_amd
