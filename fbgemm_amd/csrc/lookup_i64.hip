// One instance of the general pooled-lookup kernel.
#include "lookup_general.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LOOKUP_LAUNCH(launch_lookup_i64, int64_t, false)
} // namespace fbgemm_amd
