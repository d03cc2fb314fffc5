// Bare streaming kernels with the load/store policy of the normalisation kernels and no
// arithmetic: what one-read-one-write and two-reads-one-write traffic reaches on the machine at
// hand.  Measurement aid for benchmarks; the product kernels do not use them.
#pragma once
#include "common.hpp"

namespace tt {

constexpr int kProbeThreads = 512;

// out[i] = a[i] (TWO == false) or a[i] ^ b[i] (TWO == true) over n 128-bit packs; grid-stride,
// U packs per lane in flight.
template <bool TWO, int U>
__global__ void __launch_bounds__(kProbeThreads) stream_probe(void* __restrict__ out, const void* __restrict__ a,
                                                             const void* __restrict__ b, size_t n) {
  const size_t stride = (size_t)gridDim.x * kProbeThreads;
  for (size_t i = (size_t)blockIdx.x * kProbeThreads + threadIdx.x; i < n; i += U * stride) {
    u32x4 va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = i + u * stride;
      if (j < n) {
        va[u] = load_stream(a, j * kPack);
        if (TWO) vb[u] = load_stream(b, j * kPack);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = i + u * stride;
      if (j < n) store_stream(out, j * kPack, TWO ? (va[u] ^ vb[u]) : va[u]);
    }
  }
}

}  // namespace tt
