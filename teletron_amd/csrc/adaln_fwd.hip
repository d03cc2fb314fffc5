// Instantiates the adaln fwd kernel family (one translation unit per family so they build in parallel).
#include "kernel_table.hpp"

namespace tt {
KernelInfo adaln_fwd_kernel(bool narrow, int idx, bool full) { return lookup_fwd<kAdaLN>(narrow, idx, full); }
}  // namespace tt
