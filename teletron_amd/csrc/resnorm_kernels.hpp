// Residual update fused with the normalisation that follows it (wide rows only):
//
//   s = x + gate * r            (GATED)   or   s = x + r
//   y = LayerNorm(s) * (one + scale) + shift
//
// `one` is 1 for AdaLN modulation and 0 for an affine LayerNorm (scale = weight, shift = bias).
// Both s (the new residual stream, rounded to bf16 before it is normalised, as the unfused
// sequence would) and y are written, so the pair costs 8 bytes per element instead of the
// 6 + 4 of a residual kernel followed by a normalisation kernel.
//
// Backward takes the gradients arriving at both outputs and returns their sum at s:
//
//   ds = ds_in + dLayerNorm(dy)          -> dx  (and dr when there is no gate)
//   dr = gate * ds,   dgate = sum_rows ds * r          (GATED)
//   dscale = sum_rows dy * x_hat,   dshift = sum_rows dy
//
// 8 (ungated) or 12 (gated) bytes per element instead of the 6 + 6 (+ 6) of a normalisation
// backward, a gradient accumulation and a gate backward.  Same skeleton as norm_kernels.hpp.
#pragma once
#include "norm_kernels.hpp"

namespace tt {

struct ResFwdArgs {
  void* s;             // out [rows, cols] bf16
  void* y;             // out [rows, cols] bf16
  const void* x;
  const void* r;
  const void* gate;    // [B or 1, cols] bf16 (GATED kernels)
  const void* scale;   // [B or 1, cols] bf16
  const void* shift;   // [B or 1, cols] bf16
  float* mean;         // optional [rows]
  float* rstd;         // optional [rows]
  int64_t rows_per_batch;
  int64_t n_tiles;
  int64_t gate_stride;   // elements between the gate vectors of consecutive batches: cols or 0
  int64_t param_stride;  // same for scale / shift
  int cols;
  int packs;
  float eps;
  float inv_cols;
  float one;
};

struct ResBwdArgs {
  void* dx;            // out [rows, cols] bf16: ds
  void* dr;            // out [rows, cols] bf16: gate * ds (GATED kernels)
  const void* dy;      // gradient of y
  const void* ds_in;   // gradient arriving at s from its other consumers; may be null (zero)
  const void* s;       // saved forward output s
  const void* r;       // (GATED kernels)
  const void* gate;    // (GATED kernels)
  const void* scale;
  float* partials;     // [B][gridDim.x][NACC][C]: dscale, dshift, (GATED) dgate
  int64_t rows_per_batch;
  int64_t n_tiles;
  int64_t gate_stride;
  int64_t param_stride;
  int cols;
  int packs;
  float eps;
  float inv_cols;
  float one;
};

// Epilogue: fold the Q row groups of the workgroup into group 0 (group order, through LDS) and
// write the workgroup's NACC partial column sums.
template <int NACC, int W, int P, int Q>
__device__ __forceinline__ void wide_write_partials_n(float (&acc)[NACC][P][8], const bool (&act)[P], const int (&col)[P],
                                                      float* partials, int64_t b, int C, int q, int w, int lane) {
  __shared__ __attribute__((aligned(16))) float comb[Q > 1 ? 64 * W * P * 8 : 4];
  if constexpr (Q > 1) {
#pragma unroll
    for (int n = 0; n < NACC; ++n) {
      for (int qq = 1; qq < Q; ++qq) {
        __syncthreads();
        if (q == qq) {
#pragma unroll
          for (int p = 0; p < P; ++p)
#pragma unroll
            for (int j = 0; j < 8; ++j) comb[((p * W + w) * 64 + lane) * 8 + j] = acc[n][p][j];
        }
        __syncthreads();
        if (q == 0) {
#pragma unroll
          for (int p = 0; p < P; ++p)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[n][p][j] += comb[((p * W + w) * 64 + lane) * 8 + j];
        }
      }
    }
  }
  if (q == 0) {
    float* base = partials + ((size_t)(b * gridDim.x + blockIdx.x) * NACC) * C;
#pragma unroll
    for (int n = 0; n < NACC; ++n)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        if (act[p]) {
          f32x4* d = reinterpret_cast<f32x4*>(base + (size_t)n * C + col[p]);
          d[0] = f32x4{acc[n][p][0], acc[n][p][1], acc[n][p][2], acc[n][p][3]};
          d[1] = f32x4{acc[n][p][4], acc[n][p][5], acc[n][p][6], acc[n][p][7]};
        }
      }
  }
}

// ============================================================================ forward
template <int W, int P, int R, int Q, bool FULL, bool GATED>
__global__ __launch_bounds__(64 * W * Q) void resnorm_fwd_wide(const ResFwdArgs a) {
  __shared__ float red[2][Q][W * R];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = wave / W;
  const int w = wave - q * W;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;

  int col[P];
  bool act[P];
  float g[P][8], sh[P][8], gt[GATED ? P : 1][8];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0}, r1 = {0, 0, 0, 0}, r2 = {0, 0, 0, 0};
    if (act[p]) {
      r0 = load_cached(a.scale, b * a.param_stride + col[p]);
      r1 = load_cached(a.shift, b * a.param_stride + col[p]);
      if constexpr (GATED) r2 = load_cached(a.gate, b * a.gate_stride + col[p]);
    }
    unpack8(r0, g[p]);
    unpack8(r1, sh[p]);
    if constexpr (GATED) unpack8(r2, gt[p]);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[p][j] += a.one;
  }

  u32x4 rawx[R][P], rawr[R][P];
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        rawx[r][p] = u32x4{0, 0, 0, 0};
        rawr[r][p] = u32x4{0, 0, 0, 0};
        if (r0 + r < S && act[p]) {
          const size_t off = (size_t)((b * S + r0 + r) * C + col[p]);
          rawx[r][p] = load_stream(a.x, off);
          rawr[r][p] = load_stream(a.r, off);
        }
      }
  };

  unsigned phase = 0;
  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float xf[R][P][8];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = row0 + r < S;
      const int64_t row = b * S + row0 + r;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float rf[8];
        unpack8(rawx[r][p], xf[r][p]);
        unpack8(rawr[r][p], rf);
#pragma unroll
        for (int j = 0; j < 8; ++j) xf[r][p][j] = GATED ? fmaf(gt[p][j], rf[j], xf[r][p][j]) : xf[r][p][j] + rf[j];
        // the residual stream is stored as bf16, and it is that rounded value which is normalised
        const u32x4 sp = pack8(xf[r][p]);
        if (rv[r] && act[p]) store_stream(a.s, (size_t)(row * C + col[p]), sp);
        unpack8(sp, xf[r][p]);
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);

    float mean[R];
    {
      float s[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float t = 0.f;
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
          for (int j = 0; j < 8; ++j) t += xf[r][p][j];
        s[r] = t;
      }
      rowgroup_allsum<W, R>(s, red[phase & 1][q], w, lane);
      ++phase;
#pragma unroll
      for (int r = 0; r < R; ++r) mean[r] = s[r] * a.inv_cols;
    }

    float v[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float t = 0.f;
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float d = xf[r][p][j] - mean[r];
          if constexpr (!FULL) d = act[p] ? d : 0.f;
          xf[r][p][j] = d;
          t = fmaf(d, d, t);
        }
      v[r] = t;
    }
    rowgroup_allsum<W, R>(v, red[phase & 1][q], w, lane);
    ++phase;

#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float rstd = rsqrtf(v[r] * a.inv_cols + a.eps);
      if (rv[r]) {
        const int64_t row = b * S + row0 + r;
#pragma unroll
        for (int p = 0; p < P; ++p) {
          if (act[p]) {
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = fmaf(xf[r][p][j] * rstd, g[p][j], sh[p][j]);
            store_stream(a.y, (size_t)(row * C + col[p]), pack8(o));
          }
        }
        if (w == 0 && lane == 0) {
          if (a.mean) a.mean[row] = mean[r];
          if (a.rstd) a.rstd[row] = rstd;
        }
      }
    }
  }
}

// ============================================================================ backward
template <int W, int P, int R, int Q, bool FULL, bool GATED>
__global__ __launch_bounds__(64 * W * Q) void resnorm_bwd_wide(const ResBwdArgs a) {
  constexpr int NACC = GATED ? 3 : 2;
  constexpr int NV = 3;
  __shared__ float red[2][Q][W * R * NV];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = wave / W;
  const int w = wave - q * W;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;
  const bool have_ds = a.ds_in != nullptr;

  int col[P];
  bool act[P];
  float g[P][8], gt[GATED ? P : 1][8];
  float acc[NACC][P][8];   // dscale, dshift, (GATED) dgate
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0}, r2 = {0, 0, 0, 0};
    if (act[p]) {
      r0 = load_cached(a.scale, b * a.param_stride + col[p]);
      if constexpr (GATED) r2 = load_cached(a.gate, b * a.gate_stride + col[p]);
    }
    unpack8(r0, g[p]);
    if constexpr (GATED) unpack8(r2, gt[p]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      g[p][j] += a.one;
#pragma unroll
      for (int n = 0; n < NACC; ++n) acc[n][p][j] = 0.f;
    }
  }

  u32x4 raws[R][P], rawd[R][P], rawg[R][P], rawr[GATED ? R : 1][GATED ? P : 1];
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        raws[r][p] = u32x4{0, 0, 0, 0};
        rawd[r][p] = u32x4{0, 0, 0, 0};
        rawg[r][p] = u32x4{0, 0, 0, 0};
        if constexpr (GATED) rawr[r][p] = u32x4{0, 0, 0, 0};
        if (r0 + r < S && act[p]) {
          const size_t off = (size_t)((b * S + r0 + r) * C + col[p]);
          raws[r][p] = load_stream(a.s, off);
          rawd[r][p] = load_stream(a.dy, off);
          if (have_ds) rawg[r][p] = load_stream(a.ds_in, off);
          if constexpr (GATED) rawr[r][p] = load_stream(a.r, off);
        }
      }
  };

  unsigned phase = 0;
  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float xf[R][P][8], df[R][P][8];
    u32x4 keepg[R][P], keepr[GATED ? R : 1][GATED ? P : 1];   // still packed: unpacked where they are used
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = row0 + r < S;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        unpack8(raws[r][p], xf[r][p]);
        unpack8(rawd[r][p], df[r][p]);
        keepg[r][p] = rawg[r][p];
        if constexpr (GATED) keepr[r][p] = rawr[r][p];
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);

    float mean[R];
    {
      float s[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float t = 0.f;
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
          for (int j = 0; j < 8; ++j) t += xf[r][p][j];
        s[r] = t;
      }
      rowgroup_allsum<W, R>(s, red[phase & 1][q], w, lane);
      ++phase;
#pragma unroll
      for (int r = 0; r < R; ++r) mean[r] = s[r] * a.inv_cols;
    }

    float red_v[R * NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float sv = 0.f, sh_ = 0.f, sg = 0.f;
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float d = xf[r][p][j] - mean[r];
          if constexpr (!FULL) d = act[p] ? d : 0.f;
          xf[r][p][j] = d;
          const float gg = df[r][p][j] * g[p][j];
          sv = fmaf(d, d, sv);
          sh_ = fmaf(gg, d, sh_);
          sg += gg;
        }
      red_v[r * NV + 0] = sv;
      red_v[r * NV + 1] = sh_;
      red_v[r * NV + 2] = sg;
    }
    rowgroup_allsum<W, R * NV>(red_v, red[phase & 1][q], w, lane);
    ++phase;

#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float rstd = rv[r] ? rsqrtf(red_v[r * NV + 0] * a.inv_cols + a.eps) : 0.f;   // zero-filled padding rows stay out of the column sums
      const float k2 = -(rstd * rstd) * (red_v[r * NV + 1] * a.inv_cols);
      const float k1 = -rstd * (red_v[r * NV + 2] * a.inv_cols);
      const int64_t row = b * S + row0 + r;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float o[8], o2[8], gin[8], rf[8];
        unpack8(keepg[r][p], gin);
        if constexpr (GATED) unpack8(keepr[r][p], rf);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float xh = xf[r][p][j] * rstd;
          const float dyv = df[r][p][j];
          acc[0][p][j] = fmaf(dyv, xh, acc[0][p][j]);
          acc[1][p][j] += dyv;
          const float ds = gin[j] + fmaf(xh, k2, fmaf(dyv * g[p][j], rstd, k1));
          o[j] = ds;
          if constexpr (GATED) {
            acc[2][p][j] = fmaf(ds, rf[j], acc[2][p][j]);
            o2[j] = gt[p][j] * ds;
          }
        }
        if (rv[r] && act[p]) {
          store_stream(a.dx, (size_t)(row * C + col[p]), pack8(o));
          if constexpr (GATED) store_stream(a.dr, (size_t)(row * C + col[p]), pack8(o2));
        }
      }
    }
  }

  wide_write_partials_n<NACC, W, P, Q>(acc, act, col, a.partials, b, C, q, w, lane);
}

}  // namespace tt
