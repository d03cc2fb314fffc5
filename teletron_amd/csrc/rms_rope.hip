// Instantiates RMSNorm + rotary embedding (forward and backward; wide rows holding all heads of a
// token, and narrow rows holding one head each).
#include "kernel_table.hpp"

namespace tt {
KernelInfo rms_rope_kernel(bool narrow, bool backward, int idx, bool full, int64_t heads) {
  return lookup_rope(narrow, backward, idx, full, heads);
}
}  // namespace tt
