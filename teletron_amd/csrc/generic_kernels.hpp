// Element-wise (16-bit load/store) kernels for shapes the vector kernels do not take:
// row widths that are not a multiple of 8 and base pointers that are not 16-byte aligned.
// Correctness path, not a bandwidth path: one 256-thread workgroup per row, the row is
// re-read from cache for each pass, parameter gradients come from a second kernel that
// walks the rows column by column with the row statistics saved by the first.
#pragma once
#include "common.hpp"
#include "norm_kernels.hpp"

namespace tt {

constexpr int kGenThreads = 256;

// Sum over the 256 threads of a workgroup; every thread gets the total.  `buf` holds
// 4 floats and may be reused after the call returns (trailing barrier).
__device__ __forceinline__ float block256_allsum(float v, float* buf) {
  v = wave_allsum(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) buf[wave] = v;
  __syncthreads();
  const float t = (buf[0] + buf[1]) + (buf[2] + buf[3]);
  __syncthreads();
  return t;
}

struct GenFwdArgs {
  uint16_t* y; const uint16_t* x; const uint16_t* p0; const uint16_t* p1;
  float* mean; float* rstd; uint16_t* x_norm;
  int64_t rows, rows_per_batch; int cols; float eps, inv_cols;
};

template <int KIND>
__global__ __launch_bounds__(kGenThreads) void norm_fwd_generic(const GenFwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  __shared__ float buf[4];
  const int C = a.cols;
  for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
    const uint16_t* xr = a.x + row * C;
    const int64_t pb = ADALN ? (row / a.rows_per_batch) * C : 0;
    float mean = 0.f;
    if constexpr (ADALN) {
      float s = 0.f;
      for (int c = threadIdx.x; c < C; c += kGenThreads) s += bf16_to_f32(xr[c]);
      mean = block256_allsum(s, buf) * a.inv_cols;
    }
    float v = 0.f;
    for (int c = threadIdx.x; c < C; c += kGenThreads) {
      const float d = bf16_to_f32(xr[c]) - mean;
      v = fmaf(d, d, v);
    }
    const float rstd = rsqrtf(block256_allsum(v, buf) * a.inv_cols + a.eps);
    for (int c = threadIdx.x; c < C; c += kGenThreads) {
      const float xh = (bf16_to_f32(xr[c]) - mean) * rstd;
      const float g = bf16_to_f32(a.p0[pb + c]);
      const float o = ADALN ? fmaf(xh, 1.0f + g, bf16_to_f32(a.p1[pb + c])) : xh * g;
      a.y[row * C + c] = f32_to_bf16(o);
      if (a.x_norm) a.x_norm[row * C + c] = f32_to_bf16(xh);
    }
    if (threadIdx.x == 0) {
      if (ADALN && a.mean) a.mean[row] = mean;
      if (a.rstd) a.rstd[row] = rstd;
    }
  }
}

struct GenBwdArgs {
  uint16_t* dx; const uint16_t* dy; const uint16_t* x; const uint16_t* p0;
  float* stats;   // [rows][2]: mean, rstd (written by the dx kernel, read by the column kernel)
  void* out0; void* out1;   // parameter gradients [B, C]
  int64_t rows, rows_per_batch; int cols; float eps, inv_cols; int out_bf16;
};

template <int KIND>
__global__ __launch_bounds__(kGenThreads) void norm_bwd_generic(const GenBwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  __shared__ float buf[4];
  const int C = a.cols;
  for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
    const uint16_t* xr = a.x + row * C;
    const uint16_t* dr = a.dy + row * C;
    const int64_t pb = ADALN ? (row / a.rows_per_batch) * C : 0;
    float mean = 0.f;
    if constexpr (ADALN) {
      float s = 0.f;
      for (int c = threadIdx.x; c < C; c += kGenThreads) s += bf16_to_f32(xr[c]);
      mean = block256_allsum(s, buf) * a.inv_cols;
    }
    float sv = 0.f, sh = 0.f, sg = 0.f;
    for (int c = threadIdx.x; c < C; c += kGenThreads) {
      const float d = bf16_to_f32(xr[c]) - mean;
      const float p = bf16_to_f32(a.p0[pb + c]);
      const float gg = bf16_to_f32(dr[c]) * (ADALN ? 1.0f + p : p);
      sv = fmaf(d, d, sv);
      sh = fmaf(gg, d, sh);
      sg += gg;
    }
    sv = block256_allsum(sv, buf);
    sh = block256_allsum(sh, buf);
    if constexpr (ADALN) sg = block256_allsum(sg, buf);
    const float rstd = rsqrtf(sv * a.inv_cols + a.eps);
    const float k2 = -(rstd * rstd) * (sh * a.inv_cols);
    const float k1 = ADALN ? -rstd * (sg * a.inv_cols) : 0.f;
    for (int c = threadIdx.x; c < C; c += kGenThreads) {
      const float xh = (bf16_to_f32(xr[c]) - mean) * rstd;
      const float p = bf16_to_f32(a.p0[pb + c]);
      const float gg = bf16_to_f32(dr[c]) * (ADALN ? 1.0f + p : p);
      a.dx[row * C + c] = f32_to_bf16(fmaf(xh, k2, fmaf(gg, rstd, k1)));
    }
    if (threadIdx.x == 0) {
      a.stats[2 * row] = mean;
      a.stats[2 * row + 1] = rstd;
    }
  }
}

// Parameter gradients: workgroup = 64 columns x 16 row slices (blockIdx.y = batch); slice s
// takes rows s, s+16, ... of the batch; the slices are folded in slice order through LDS.
template <int KIND>
__global__ __launch_bounds__(1024) void norm_colgrad_generic(const GenBwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  __shared__ float fold[16][2][64];
  const int lane = threadIdx.x & 63;
  const int slice = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int64_t b = blockIdx.y;
  const int C = a.cols;
  float acc0 = 0.f, acc1 = 0.f;
  if (c < C) {
    for (int64_t r = slice; r < a.rows_per_batch; r += 16) {
      const int64_t row = b * a.rows_per_batch + r;
      const float mean = a.stats[2 * row], rstd = a.stats[2 * row + 1];
      const float dyv = bf16_to_f32(a.dy[row * C + c]);
      const float xh = (bf16_to_f32(a.x[row * C + c]) - mean) * rstd;
      acc0 = fmaf(dyv, xh, acc0);
      acc1 += dyv;
    }
  }
  fold[slice][0][lane] = acc0;
  fold[slice][1][lane] = acc1;
  __syncthreads();
  if (slice < (ADALN ? 2 : 1) && c < C) {
    float t = fold[0][slice][lane];
#pragma unroll
    for (int s = 1; s < 16; ++s) t += fold[s][slice][lane];
    void* out = slice == 0 ? a.out0 : a.out1;
    const size_t idx = (size_t)b * C + c;
    if (a.out_bf16) static_cast<uint16_t*>(out)[idx] = f32_to_bf16(t);
    else            static_cast<float*>(out)[idx] = t;
  }
}

}  // namespace tt
