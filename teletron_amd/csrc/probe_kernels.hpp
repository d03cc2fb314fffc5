// Bare streaming kernels with the load/store policy of the normalisation kernels and no
// arithmetic: what one-read-one-write and two-reads-one-write traffic, and reads or writes on
// their own, reach on the machine at hand.  Measurement aid for benchmarks; the product kernels
// do not use them.
#pragma once
#include "common.hpp"

namespace tt {

constexpr int kProbeMaxThreads = 512;

enum ProbeMode : int { kProbeCopy = 0, kProbeXor = 1, kProbeRead = 2, kProbeWrite = 3 };

// Over n 128-bit packs, grid-stride, U packs per lane in flight, any workgroup size up to
// kProbeMaxThreads:
//   kProbeCopy   out[i] = a[i]
//   kProbeXor    out[i] = a[i] ^ b[i]
//   kProbeRead   a[i] is loaded and dropped (the empty asm keeps the load and its wait alive)
//   kProbeWrite  out[i] = the pack's index, low 32 bits, in each of its four words
template <int MODE, int U>
__global__ void __launch_bounds__(kProbeMaxThreads) stream_probe(void* __restrict__ out, const void* __restrict__ a,
                                                             const void* __restrict__ b, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += U * stride) {
    u32x4 va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = i + u * stride;
      const unsigned w = (unsigned)j;
      va[u] = u32x4{w, w, w, w};
      vb[u] = u32x4{0, 0, 0, 0};
      if (j < n) {
        if (MODE != kProbeWrite) va[u] = load_stream(a, j * kPack);
        if (MODE == kProbeXor) vb[u] = load_stream(b, j * kPack);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = i + u * stride;
      if (MODE == kProbeRead) asm volatile("" ::"v"(va[u]));
      else if (j < n) store_stream(out, j * kPack, va[u] ^ vb[u]);
    }
  }
}

// One read, two writes: out0[i] = a[i], out1[i] = ~a[i] (the traffic of a forward that also saves
// a second tensor).  Persistent tile loop with the next tile prefetched, U packs per lane; a tile's
// stores go to out0 first, then to out1.
template <int U>
__global__ void __launch_bounds__(kProbeMaxThreads) stream_probe_two_outputs(void* __restrict__ out0, void* __restrict__ out1,
                                                                         const void* __restrict__ a, size_t n) {
  const size_t T = blockDim.x, tile = T * U;
  const size_t n_tiles = (n + tile - 1) / tile;
  u32x4 raw[U];
  auto fetch = [&](size_t t) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = t * tile + u * T + threadIdx.x;
      raw[u] = u32x4{0, 0, 0, 0};
      if (j < n) raw[u] = load_stream(a, j * kPack);
    }
  };
  size_t t = blockIdx.x;
  if (t < n_tiles) fetch(t);
  for (; t < n_tiles; t += gridDim.x) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = raw[u];
    if (t + gridDim.x < n_tiles) fetch(t + gridDim.x);
    __syncthreads();   // lock-step only
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = t * tile + u * T + threadIdx.x;
      if (j < n) store_stream(out0, j * kPack, v[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t j = t * tile + u * T + threadIdx.x;
      if (j < n) store_stream(out1, j * kPack, ~v[u]);
    }
  }
}

}  // namespace tt
