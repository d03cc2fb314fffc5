// Instantiates the adaln bwd saved kernel family: backward from the tensors the reference saves
// (x_norm / forward output + rstd).  One translation unit per family so they build in parallel.
#include "kernel_table.hpp"

namespace tt {
KernelInfo adaln_bwd_saved_kernel(bool narrow, int idx, bool full) { return lookup_bwd_saved<kAdaLN>(narrow, idx, full); }
}  // namespace tt
