// Instantiates the rms fwd kernel family (one translation unit per family so they build in parallel).
#include "kernel_table.hpp"

namespace tt {
KernelInfo rms_fwd_kernel(bool narrow, int idx, bool full) { return lookup_fwd<kRMS>(narrow, idx, full); }
}  // namespace tt
