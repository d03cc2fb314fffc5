// Instantiates the adaln fwd kernel family that also stores x_norm (one translation unit per family so they build in parallel).
#include "kernel_table.hpp"

namespace tt {
KernelInfo adaln_fwd_xnorm_kernel(bool narrow, int idx, bool full) { return lookup_fwd_xn(narrow, idx, full); }
}  // namespace tt
