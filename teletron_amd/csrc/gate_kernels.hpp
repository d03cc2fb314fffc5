// Gated residual add, the op that follows every fused AdaLN site in the DiT blocks:
//   forward   out = x + gate * residual                      (gate broadcast over the rows of a batch)
//   backward  dresidual = dout * gate,  dgate[b, c] = sum_rows dout * residual   (dx = dout, no kernel)
// Two streamed inputs and one streamed output, no row statistics: the same column-ownership
// skeleton as the normalisation backward kernels (see norm_kernels.hpp) without the reductions.
#pragma once
#include "norm_kernels.hpp"

namespace tt {

struct GateArgs {
  void* out;         // forward: out;            backward: dresidual
  const void* a;     // forward: x;              backward: dout
  const void* b;     // forward: residual;       backward: residual
  const void* gate;  // [B, C] bf16
  float* partials;   // backward: [B][gridDim.x][1][C]
  int64_t rows_per_batch;
  int64_t n_tiles;
  int cols;
  int packs;
};

enum GateMode : int { kGateFwd = 0, kGateBwd = 1 };

template <int MODE, int W, int P, int R, int Q, bool FULL>
__global__ __launch_bounds__(64 * W * Q) void gate_wide(const GateArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = wave / W;
  const int w = wave - q * W;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;

  int col[P];
  bool act[P];
  float g[P][8], acc0[P][8], acc1[P][8];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0};
    if (act[p]) r0 = load_cached(a.gate, b * C + col[p]);
    unpack8(r0, g[p]);
#pragma unroll
    for (int j = 0; j < 8; ++j) { acc0[p][j] = 0.f; acc1[p][j] = 0.f; }
  }

  u32x4 rawa[R][P], rawb[R][P];
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        rawa[r][p] = u32x4{0, 0, 0, 0};
        rawb[r][p] = u32x4{0, 0, 0, 0};
        if (r0 + r < S && act[p]) {
          const size_t off = (size_t)((b * S + r0 + r) * C + col[p]);
          rawa[r][p] = load_stream(a.a, off);
          rawb[r][p] = load_stream(a.b, off);
        }
      }
  };

  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float af[R][P][8], bf[R][P][8];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        unpack8(rawa[r][p], af[r][p]);
        unpack8(rawb[r][p], bf[r][p]);
      }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);
    // Keeps the waves of the workgroup in step, which the memory system rewards (a denser,
    // narrower request stream); nothing is exchanged here.
    if constexpr (W * Q > 1) __syncthreads();
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = b * S + row0 + r;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if constexpr (MODE == kGateFwd) {
            o[j] = fmaf(g[p][j], bf[r][p][j], af[r][p][j]);
          } else {
            o[j] = af[r][p][j] * g[p][j];
            acc0[p][j] = fmaf(af[r][p][j], bf[r][p][j], acc0[p][j]);
          }
        }
        if (row0 + r < S && act[p]) store_stream(a.out, (size_t)(row * C + col[p]), pack8(o));
      }
    }
  }
  if constexpr (MODE == kGateBwd)
    wide_write_partials<false, W, P, Q>(acc0, acc1, act, col, a.partials, b, C, q, w, lane);
}

template <int MODE, int L, int R, int NW, bool FULL>
__global__ __launch_bounds__(64 * NW) void gate_narrow(const GateArgs a) {
  constexpr int RPW = 64 / L;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int pi = lane & (L - 1);
  const int ri = lane / L;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;
  const bool act = FULL || pi < a.packs;
  const int col = pi * kPack;

  float g[8], acc0[8], acc1[8];
  {
    u32x4 r0 = {0, 0, 0, 0};
    if (act) r0 = load_cached(a.gate, b * C + col);
    unpack8(r0, g);
#pragma unroll
    for (int j = 0; j < 8; ++j) { acc0[j] = 0.f; acc1[j] = 0.f; }
  }

  u32x4 rawa[R], rawb[R];
  auto fetch = [&](int64_t t) {
    const int64_t rb = t * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t rr = rb + r * RPW;
      rawa[r] = u32x4{0, 0, 0, 0};
      rawb[r] = u32x4{0, 0, 0, 0};
      if (rr < S && act) {
        const size_t off = (size_t)((b * S + rr) * C + col);
        rawa[r] = load_stream(a.a, off);
        rawb[r] = load_stream(a.b, off);
      }
    }
  };

  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t rbase = tile * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
    float af[R][8], bf[R][8];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      unpack8(rawa[r], af[r]);
      unpack8(rawb[r], bf[r]);
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);
    if constexpr (NW > 1) __syncthreads();   // lock-step only, as in gate_wide
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if constexpr (MODE == kGateFwd) {
          o[j] = fmaf(g[j], bf[r][j], af[r][j]);
        } else {
          o[j] = af[r][j] * g[j];
          acc0[j] = fmaf(af[r][j], bf[r][j], acc0[j]);
        }
      }
      const int64_t rr = rbase + r * RPW;
      if (rr < S && act) store_stream(a.out, (size_t)((b * S + rr) * C + col), pack8(o));
    }
  }
  if constexpr (MODE == kGateBwd)
    narrow_write_partials<false, L, NW>(acc0, acc1, a.partials, b, C, pi, ri, wave);
}

}  // namespace tt
