// One instance of the general pooled-lookup kernel.
#include "lookup_general.h"

namespace fbgemm_amd {
FBGEMM_AMD_DEFINE_LOOKUP_LAUNCH(launch_lookup_i32_general, int32_t, true)
} // namespace fbgemm_amd
