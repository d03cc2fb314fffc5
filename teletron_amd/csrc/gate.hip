// Instantiates the gated-residual kernel family (forward and backward).
#include "kernel_table.hpp"

namespace tt {
KernelInfo gate_fwd_kernel(bool narrow, int idx, bool full) { return lookup_gate<kGateFwd>(narrow, idx, full); }
KernelInfo gate_bwd_kernel(bool narrow, int idx, bool full) { return lookup_gate<kGateBwd>(narrow, idx, full); }
}  // namespace tt
