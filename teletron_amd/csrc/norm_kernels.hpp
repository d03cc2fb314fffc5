// Streaming kernels for fused AdaLN / RMSNorm, forward and backward, on gfx950.
//
// Two shapes of kernel cover every row width that is a multiple of 8:
//
//  * "wide"   (more than 32 packs per row): a row is owned by a *row group* of
//    W waves; lane l of wave w owns the packs  p*64*W + w*64 + l  (p < P), so
//    each load instruction of a wave is one contiguous 1 KiB segment.  A
//    workgroup holds Q row groups and walks the rows of one batch in tiles of
//    Q*R rows.  The row stays in registers between the statistics pass and the
//    output pass, so x (and dy) are read from HBM exactly once.
//  * "narrow" (at most 32 packs per row): L = 2^k lanes own one row, a wave
//    carries 64/L rows per load and the row reductions never leave the wave.
//
// Column ownership is fixed for the lifetime of a workgroup.  The parameters a
// lane needs therefore live in registers as fp32, and in backward the lane's
// share of dscale/dshift/dgamma is accumulated in fp32 registers over all rows
// the workgroup visits, then written once as a per-workgroup partial.  A second
// kernel (reduce_partials) sums the partials in a fixed order: no atomics, so
// the parameter gradients are bitwise reproducible.
#pragma once
#include "common.hpp"

namespace tt {

enum Kind : int { kAdaLN = 0, kRMS = 1 };

// Software prefetch of the next tile (see the kernels): without it the kernels are 8-10 % slower.
constexpr bool PF = true;

struct FwdArgs {
  void* y;
  const void* x;
  const void* p0;   // AdaLN: scale [B, C];  RMSNorm: weight [C]
  const void* p1;   // AdaLN: shift [B, C];  RMSNorm: unused
  float* mean;      // optional [rows]
  float* rstd;      // optional [rows]
  void* x_norm;     // [rows, cols] bf16: the normalised input before modulation (XN kernels only)
  int64_t rows_per_batch;
  int64_t n_tiles;  // tiles per batch
  int cols;
  int packs;        // cols / 8
  float eps;
  float inv_cols;
  // rotary embedding fused behind RMSNorm (ROPE kernels only): (cos, sin) per position and
  // complex index of a head, fp32 [seq_len][head_dim / 2][2]; row r sits at position r % seq_len
  const float* freqs;
  int64_t seq_len;
  int head_dim;
  int64_t rows_per_pos;   // narrow ROPE kernels: consecutive rows (heads) that share one position
};

struct BwdArgs {
  void* dx;
  const void* dy;
  const void* x;
  const void* p0;    // AdaLN: scale [B, C];  RMSNorm: weight [C]
  float* partials;   // [B][gridDim.x][NACC][C]
  int64_t rows_per_batch;
  int64_t n_tiles;
  int cols;
  int packs;
  float eps;
  float inv_cols;
  const float* freqs;   // as in FwdArgs (ROPE kernels only)
  int64_t seq_len;
  int head_dim;
  int64_t rows_per_pos;
};

// Rotary helpers: a pack holds 4 (re, im) pairs; fr holds their 4 (cos, sin) pairs.
__device__ __forceinline__ void rope_rotate(float (&v)[8], const float (&fr)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float re = v[2 * k], im = v[2 * k + 1], c = fr[2 * k], sn = fr[2 * k + 1];
    v[2 * k] = fmaf(re, c, -im * sn);
    v[2 * k + 1] = fmaf(re, sn, im * c);
  }
}
// Multiplication by the conjugate: the gradient of rope_rotate with respect to its input.
__device__ __forceinline__ void rope_unrotate(float (&v)[8], const float (&fr)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float re = v[2 * k], im = v[2 * k + 1], c = fr[2 * k], sn = fr[2 * k + 1];
    v[2 * k] = fmaf(re, c, im * sn);
    v[2 * k + 1] = fmaf(im, c, -re * sn);
  }
}
__device__ __forceinline__ void load_freq8(const float* freqs, size_t off, float (&fr)[8]) {
  const f32x4* p = reinterpret_cast<const f32x4*>(freqs + off);
  const f32x4 a = p[0], b = p[1];
  fr[0] = a[0]; fr[1] = a[1]; fr[2] = a[2]; fr[3] = a[3];
  fr[4] = b[0]; fr[5] = b[1]; fr[6] = b[2]; fr[7] = b[3];
}

// Sum NV values over the W waves of one row group.  `buf` points at W*NV floats
// of LDS private to (reduction phase parity, row group).  Callers alternate two
// buffers between consecutive reductions, which makes one barrier per reduction
// sufficient: a wave can only overwrite a buffer after passing the barrier of
// the reduction in between, which every wave reaches after its reads.
template <int W, int NV>
__device__ __forceinline__ void rowgroup_allsum(float (&v)[NV], float* buf, int w, int lane) {
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = wave_allsum(v[i]);
  if constexpr (W > 1) {
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < NV; ++i) buf[w * NV + i] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float t = buf[i];
#pragma unroll
      for (int ww = 1; ww < W; ++ww) t += buf[ww * NV + i];
      v[i] = t;
    }
  }
}

// ============================================================================ wide forward
// XN: also store the normalised input before modulation (a.x_norm), paired with the y store.
template <int KIND, int W, int P, int R, int Q, bool FULL, bool ROPE = false, bool XN = false>
__global__ __launch_bounds__(64 * W * Q) void norm_fwd_wide(const FwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  static_assert(!ROPE || KIND == kRMS, "rotary embedding is fused behind RMSNorm only");
  static_assert(!XN || ADALN, "x_norm is an output of the AdaLN forward only");
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
  float g[P][8], sh[P][8];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0}, r1 = {0, 0, 0, 0};
    if (act[p]) {
      r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col[p]);
      if constexpr (ADALN) r1 = load_cached(a.p1, b * C + col[p]);
    }
    unpack8(r0, g[p]);
    unpack8(r1, sh[p]);
    if constexpr (ADALN) {
#pragma unroll
      for (int j = 0; j < 8; ++j) g[p][j] += 1.0f;
    }
  }

  // Raw packs of the tile being fetched.  With PF the loads of the next tile are
  // issued before the arithmetic of the current one, so every wave keeps a tile
  // in flight while it computes.
  u32x4 raw[R][P];
  // ROPE: the (cos, sin) table of a row (head_dim floats, at most 256) is fetched once per row
  // group by the first head_dim/4 lanes of its first wave, prefetched like the row itself, and
  // handed to the other lanes through LDS: it is written before the barrier of the row
  // reduction and read after it, two buffers alternating from tile to tile.
  __shared__ __attribute__((aligned(16))) float ftab[ROPE ? 2 : 1][ROPE ? Q : 1][ROPE ? R : 1][ROPE ? 256 : 4];
  f32x4 fq[R];
  int fcol[P];                               // column inside its head
  const bool floader = ROPE && w == 0 && lane * 4 < a.head_dim;
  // Position of the first row of the tile that fetch() takes next, kept incrementally:
  // tiles are fetched in the order blockIdx.x, blockIdx.x + gridDim.x, ...
  int64_t fpos = 0, fstep = 0;
  if constexpr (ROPE) {
#pragma unroll
    for (int p = 0; p < P; ++p) fcol[p] = col[p] % a.head_dim;
    fpos = (b * S + (int64_t)blockIdx.x * (Q * R) + q * R) % a.seq_len;
    fstep = ((int64_t)gridDim.x * (Q * R)) % a.seq_len;
  }
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
    if constexpr (ROPE) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        int64_t pos = fpos + r;
        while (pos >= a.seq_len) pos -= a.seq_len;
        fq[r] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (floader && r0 + r < S)
          fq[r] = *reinterpret_cast<const f32x4*>(a.freqs + (size_t)(pos * a.head_dim + lane * 4));
      }
      fpos += fstep;
      if (fpos >= a.seq_len) fpos -= a.seq_len;
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        raw[r][p] = u32x4{0, 0, 0, 0};
        if (r0 + r < S && act[p]) raw[r][p] = load_stream(a.x, (size_t)((b * S + r0 + r) * C + col[p]));
      }
  };

  unsigned phase = 0;
  unsigned tpar = 0;
  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x, tpar ^= 1u) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float xf[R][P][8];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = row0 + r < S;
#pragma unroll
      for (int p = 0; p < P; ++p) unpack8(raw[r][p], xf[r][p]);
    }
    if constexpr (ROPE) {
      if (floader) {
#pragma unroll
        for (int r = 0; r < R; ++r) *reinterpret_cast<f32x4*>(&ftab[tpar][q][r][lane * 4]) = fq[r];
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);

    float mean[R];
#pragma unroll
    for (int r = 0; r < R; ++r) mean[r] = 0.f;
    if constexpr (ADALN) {
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
          float d = xf[r][p][j];
          if constexpr (ADALN) {
            d -= mean[r];
            if constexpr (!FULL) d = act[p] ? d : 0.f;
            xf[r][p][j] = d;
          }
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
            float o[8], n[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float xh = xf[r][p][j] * rstd;
              n[j] = xh;
              o[j] = ADALN ? fmaf(xh, g[p][j], sh[p][j]) : xh * g[p][j];
            }
            if constexpr (ROPE) {
              float fc[8];
              const f32x4* ft = reinterpret_cast<const f32x4*>(&ftab[tpar][q][r][fcol[p]]);
              const f32x4 f0 = ft[0], f1 = ft[1];
              fc[0] = f0[0]; fc[1] = f0[1]; fc[2] = f0[2]; fc[3] = f0[3];
              fc[4] = f1[0]; fc[5] = f1[1]; fc[6] = f1[2]; fc[7] = f1[3];
              rope_rotate(o, fc);
            }
            if constexpr (XN) store_stream2(a.y, a.x_norm, (size_t)(row * C + col[p]), pack8(o), pack8(n));
            else              store_stream(a.y, (size_t)(row * C + col[p]), pack8(o));
          }
        }
        if (w == 0 && lane == 0) {
          if (ADALN && a.mean) a.mean[row] = mean[r];
          if (a.rstd) a.rstd[row] = rstd;
        }
      }
    }
  }
}

// Epilogue of the wide backward kernels: fold the Q row groups of the workgroup into
// group 0 (in group order, through LDS) and write the workgroup's partial column sums.
template <bool ADALN, int W, int P, int Q>
__device__ __forceinline__ void wide_write_partials(float (&acc0)[P][8], float (&acc1)[P][8], const bool (&act)[P],
                                                    const int (&col)[P], float* partials, int64_t b, int C,
                                                    int q, int w, int lane) {
  constexpr int NACC = ADALN ? 2 : 1;
  __shared__ __attribute__((aligned(16))) float comb[Q > 1 ? 64 * W * P * 8 : 4];
  if constexpr (Q > 1) {
#pragma unroll
    for (int acc = 0; acc < NACC; ++acc) {
      for (int qq = 1; qq < Q; ++qq) {
        __syncthreads();
        if (q == qq) {
#pragma unroll
          for (int p = 0; p < P; ++p)
#pragma unroll
            for (int j = 0; j < 8; ++j)
              comb[((p * W + w) * 64 + lane) * 8 + j] = acc == 0 ? acc0[p][j] : acc1[p][j];
        }
        __syncthreads();
        if (q == 0) {
#pragma unroll
          for (int p = 0; p < P; ++p)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float t = comb[((p * W + w) * 64 + lane) * 8 + j];
              if (acc == 0) acc0[p][j] += t; else acc1[p][j] += t;
            }
        }
      }
    }
  }
  if (q == 0) {
    float* base = partials + ((size_t)(b * gridDim.x + blockIdx.x) * NACC) * C;
#pragma unroll
    for (int p = 0; p < P; ++p) {
      if (act[p]) {
        f32x4* d0 = reinterpret_cast<f32x4*>(base + col[p]);
        d0[0] = f32x4{acc0[p][0], acc0[p][1], acc0[p][2], acc0[p][3]};
        d0[1] = f32x4{acc0[p][4], acc0[p][5], acc0[p][6], acc0[p][7]};
        if constexpr (ADALN) {
          f32x4* d1 = reinterpret_cast<f32x4*>(base + C + col[p]);
          d1[0] = f32x4{acc1[p][0], acc1[p][1], acc1[p][2], acc1[p][3]};
          d1[1] = f32x4{acc1[p][4], acc1[p][5], acc1[p][6], acc1[p][7]};
        }
      }
    }
  }
}

// ============================================================================ wide backward
template <int KIND, int W, int P, int R, int Q, bool FULL, bool ROPE = false>
__global__ __launch_bounds__(64 * W * Q) void norm_bwd_wide(const BwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  static_assert(!ROPE || KIND == kRMS, "rotary embedding is fused behind RMSNorm only");
  constexpr int NACC = ADALN ? 2 : 1;
  constexpr int NV = ADALN ? 3 : 2;  // reduced values per row in the main phase
  __shared__ float red[2][Q][W * R * NV];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = wave / W;
  const int w = wave - q * W;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;

  int col[P];
  bool act[P];
  float g[P][8];
  float acc0[P][8];  // dscale / dgamma
  float acc1[P][8];  // dshift (AdaLN only)
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0};
    if (act[p]) r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col[p]);
    unpack8(r0, g[p]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (ADALN) g[p][j] += 1.0f;
      acc0[p][j] = 0.f;
      acc1[p][j] = 0.f;
    }
  }

  u32x4 rawx[R][P], rawd[R][P];
  float fr[ROPE ? R : 1][ROPE ? P : 1][8];
  int fcol[P];
  int64_t fpos = 0, fstep = 0;   // as in the forward kernel
  if constexpr (ROPE) {
#pragma unroll
    for (int p = 0; p < P; ++p) fcol[p] = col[p] % a.head_dim;
    fpos = (b * S + (int64_t)blockIdx.x * (Q * R) + q * R) % a.seq_len;
    fstep = ((int64_t)gridDim.x * (Q * R)) % a.seq_len;
  }
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
    int64_t pos[R];
    if constexpr (ROPE) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        pos[r] = fpos + r;
        while (pos[r] >= a.seq_len) pos[r] -= a.seq_len;
      }
      fpos += fstep;
      if (fpos >= a.seq_len) fpos -= a.seq_len;
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int p = 0; p < P; ++p) {
        rawx[r][p] = u32x4{0, 0, 0, 0};
        rawd[r][p] = u32x4{0, 0, 0, 0};
        if constexpr (ROPE) {
#pragma unroll
          for (int j = 0; j < 8; ++j) fr[r][p][j] = 0.f;
        }
        if (r0 + r < S && act[p]) {
          const size_t off = (size_t)((b * S + r0 + r) * C + col[p]);
          rawx[r][p] = load_stream(a.x, off);
          rawd[r][p] = load_stream(a.dy, off);
          if constexpr (ROPE)
            load_freq8(a.freqs, (size_t)(pos[r] * a.head_dim + fcol[p]), fr[r][p]);
        }
      }
  };

  unsigned phase = 0;
  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float xf[R][P][8], df[R][P][8];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = row0 + r < S;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        unpack8(rawx[r][p], xf[r][p]);
        unpack8(rawd[r][p], df[r][p]);
        // the incoming gradient is that of the rotated output: undo the rotation first
        if constexpr (ROPE) rope_unrotate(df[r][p], fr[r][p]);
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);

    float mean[R];
#pragma unroll
    for (int r = 0; r < R; ++r) mean[r] = 0.f;
    if constexpr (ADALN) {
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

    // One pass gives sum d^2, sum g*d and (AdaLN) sum g, with d = x - mean and g = dy * param.
    float red_v[R * NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float sv = 0.f, sh_ = 0.f, sg = 0.f;
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float d = xf[r][p][j];
          if constexpr (ADALN) {
            d -= mean[r];
            if constexpr (!FULL) d = act[p] ? d : 0.f;
            xf[r][p][j] = d;
          }
          const float gg = df[r][p][j] * g[p][j];
          sv = fmaf(d, d, sv);
          sh_ = fmaf(gg, d, sh_);
          if constexpr (ADALN) sg += gg;
        }
      red_v[r * NV + 0] = sv;
      red_v[r * NV + 1] = sh_;
      if constexpr (ADALN) red_v[r * NV + 2] = sg;
    }
    rowgroup_allsum<W, R * NV>(red_v, red[phase & 1][q], w, lane);
    ++phase;

#pragma unroll
    for (int r = 0; r < R; ++r) {
      // rows past the end of the batch (zero-filled) must stay out of the column sums even when
      // eps == 0 would turn their rstd into inf
      const float rstd = rv[r] ? rsqrtf(red_v[r * NV + 0] * a.inv_cols + a.eps) : 0.f;
      // dx = rstd*g - rstd*mean(g) - x_hat * rstd*mean(g*x_hat),  mean(g*x_hat) = rstd * sum(g*d) / C
      const float k2 = -(rstd * rstd) * (red_v[r * NV + 1] * a.inv_cols);
      const float k1 = ADALN ? -rstd * (red_v[r * NV + 2] * a.inv_cols) : 0.f;
      const int64_t row = b * S + row0 + r;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float xh = xf[r][p][j] * rstd;
          const float dyv = df[r][p][j];
          acc0[p][j] = fmaf(dyv, xh, acc0[p][j]);
          if constexpr (ADALN) acc1[p][j] += dyv;
          o[j] = fmaf(xh, k2, fmaf(dyv * g[p][j], rstd, k1));
        }
        if (rv[r] && act[p]) store_stream(a.dx, (size_t)(row * C + col[p]), pack8(o));
      }
    }
  }

  wide_write_partials<ADALN, W, P, Q>(acc0, acc1, act, col, a.partials, b, C, q, w, lane);
}

// Position of a row for the narrow ROPE kernels: one row is one head, `rows_per_pos` consecutive
// rows (the heads of a token) share position (row / rows_per_pos) % seq_len.  A lane follows rows
// row0, row0 + step, row0 + 2 step, ...; the position is kept incrementally (no division in the loop).
struct RowPos {
  int64_t head, pos;       // row = (k * seq_len + pos) * rows_per_pos + head
  int64_t dhead, dpos;     // step = dpos * rows_per_pos + dhead, dpos already reduced mod seq_len
  __device__ __forceinline__ void init(int64_t row0, int64_t step, int64_t rows_per_pos, int64_t seq_len) {
    head = row0 % rows_per_pos;
    pos = (row0 / rows_per_pos) % seq_len;
    dhead = step % rows_per_pos;
    dpos = (step / rows_per_pos) % seq_len;
  }
  __device__ __forceinline__ void advance(int64_t rows_per_pos, int64_t seq_len) {
    head += dhead;
    pos += dpos;
    if (head >= rows_per_pos) { head -= rows_per_pos; pos += 1; }
    if (pos >= seq_len) pos -= seq_len;
    if (pos >= seq_len) pos -= seq_len;
  }
};

// ============================================================================ narrow forward
// L lanes per row (one pack each), 64/L rows per wave per load, R loads in flight,
// NW independent waves per workgroup.  A tile is NW*R*(64/L) consecutive rows.
// ROPE: 0 none; 1 every row looks up its own position; 2 the R * 64/L rows a wave takes per tile
// are exactly the heads of ONE token (the caller guarantees rows_per_pos == R * 64/L), so a lane
// loads its (cos, sin) entries once per tile instead of once per row.
template <int KIND, int L, int R, int NW, bool FULL, int ROPE = 0, bool XN = false>   // XN as in norm_fwd_wide
__global__ __launch_bounds__(64 * NW) void norm_fwd_narrow(const FwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  static_assert(!ROPE || KIND == kRMS, "rotary embedding is fused behind RMSNorm only");
  static_assert(!XN || ADALN, "x_norm is an output of the AdaLN forward only");
  constexpr int NF = ROPE == 1 ? R : 1;   // table entries held per lane
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

  float g[8], sh[8];
  {
    u32x4 r0 = {0, 0, 0, 0}, r1 = {0, 0, 0, 0};
    if (act) {
      r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col);
      if constexpr (ADALN) r1 = load_cached(a.p1, b * C + col);
    }
    unpack8(r0, g);
    unpack8(r1, sh);
    if constexpr (ADALN) {
#pragma unroll
      for (int j = 0; j < 8; ++j) g[j] += 1.0f;
    }
  }

  u32x4 raw[R];
  // ROPE: the 4 (cos, sin) pairs of this lane's pack at the row's position travel with the row.
  float fr[NF][8];
  RowPos rp[NF];
  if constexpr (ROPE) {
#pragma unroll
    for (int r = 0; r < NF; ++r)
      rp[r].init(b * S + (int64_t)blockIdx.x * (NW * R * RPW) + (int64_t)wave * (R * RPW) + (ROPE == 1 ? ri + r * RPW : 0),
                 (int64_t)gridDim.x * (NW * R * RPW), a.rows_per_pos, a.seq_len);
  }
  auto fetch = [&](int64_t t) {
    const int64_t rb = t * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t rr = rb + r * RPW;
      raw[r] = u32x4{0, 0, 0, 0};
      const bool table = ROPE == 1 || (ROPE == 2 && r == 0);   // this load carries table entries with it
      const int f = ROPE == 1 ? r : 0;
      if (table) {
#pragma unroll
        for (int j = 0; j < 8; ++j) fr[f][j] = 0.f;
      }
      if (rr < S && act) {
        raw[r] = load_stream(a.x, (size_t)((b * S + rr) * C + col));
        if (table) load_freq8(a.freqs, (size_t)(rp[f].pos * a.head_dim + col), fr[f]);
      }
      if (table) rp[f].advance(a.rows_per_pos, a.seq_len);
    }
  };

  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t rbase = tile * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
    float xf[R][8];
    float fc[NF][8];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = rbase + r * RPW < S;
      unpack8(raw[r], xf[r]);
      if (ROPE == 1 || (ROPE == 2 && r == 0)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) fc[ROPE == 1 ? r : 0][j] = fr[ROPE == 1 ? r : 0][j];
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float mean = 0.f;
      if constexpr (ADALN) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) t += xf[r][j];
        mean = group_allsum<L>(t) * a.inv_cols;
      }
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float d = xf[r][j];
        if constexpr (ADALN) {
          d -= mean;
          if constexpr (!FULL) d = act ? d : 0.f;
          xf[r][j] = d;
        }
        v = fmaf(d, d, v);
      }
      v = group_allsum<L>(v);
      const float rstd = rsqrtf(v * a.inv_cols + a.eps);
      if (rv[r] && act) {
        const int64_t row = b * S + rbase + r * RPW;
        float o[8], n[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float xh = xf[r][j] * rstd;
          n[j] = xh;
          o[j] = ADALN ? fmaf(xh, g[j], sh[j]) : xh * g[j];
        }
        if constexpr (ROPE) rope_rotate(o, fc[ROPE == 1 ? r : 0]);
        if constexpr (XN) store_stream2(a.y, a.x_norm, (size_t)(row * C + col), pack8(o), pack8(n));
        else              store_stream(a.y, (size_t)(row * C + col), pack8(o));
        if (pi == 0) {
          if (ADALN && a.mean) a.mean[row] = mean;
          if (a.rstd) a.rstd[row] = rstd;
        }
      }
    }
  }
}

// Epilogue of the narrow backward kernels: fold the 64/L row slots of each wave (lanes
// with equal pack index), then the waves through LDS, and write the partial column sums.
template <bool ADALN, int L, int NW>
__device__ __forceinline__ void narrow_write_partials(float (&acc0)[8], float (&acc1)[8], float* partials,
                                                      int64_t b, int C, int pi, int ri, int wave) {
  constexpr int NACC = ADALN ? 2 : 1;
  __shared__ __attribute__((aligned(16))) float comb[NW][NACC][L * 8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int m = L; m < 64; m <<= 1) {
      acc0[j] += __shfl_xor(acc0[j], m, 64);
      if constexpr (ADALN) acc1[j] += __shfl_xor(acc1[j], m, 64);
    }
  }
  if (ri == 0) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      comb[wave][0][pi * 8 + j] = acc0[j];
      if constexpr (ADALN) comb[wave][NACC - 1][pi * 8 + j] = acc1[j];
    }
  }
  __syncthreads();
  float* base = partials + ((size_t)(b * gridDim.x + blockIdx.x) * NACC) * C;
  for (int i = threadIdx.x; i < NACC * L * 8; i += 64 * NW) {
    const int acc = i / (L * 8);
    const int c = i - acc * (L * 8);
    if (c < C) {
      float t = comb[0][acc][c];
#pragma unroll
      for (int ww = 1; ww < NW; ++ww) t += comb[ww][acc][c];
      base[(size_t)acc * C + c] = t;
    }
  }
}

// ============================================================================ narrow backward
template <int KIND, int L, int R, int NW, bool FULL, int ROPE = 0>   // ROPE as in norm_fwd_narrow
__global__ __launch_bounds__(64 * NW) void norm_bwd_narrow(const BwdArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  static_assert(!ROPE || KIND == kRMS, "rotary embedding is fused behind RMSNorm only");
  constexpr int NF = ROPE == 1 ? R : 1;
  constexpr int NACC = ADALN ? 2 : 1;
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
    if (act) r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col);
    unpack8(r0, g);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (ADALN) g[j] += 1.0f;
      acc0[j] = 0.f;
      acc1[j] = 0.f;
    }
  }

  u32x4 rawx[R], rawd[R];
  float fr[NF][8];   // as in the forward kernel
  RowPos rp[NF];
  if constexpr (ROPE) {
#pragma unroll
    for (int r = 0; r < NF; ++r)
      rp[r].init(b * S + (int64_t)blockIdx.x * (NW * R * RPW) + (int64_t)wave * (R * RPW) + (ROPE == 1 ? ri + r * RPW : 0),
                 (int64_t)gridDim.x * (NW * R * RPW), a.rows_per_pos, a.seq_len);
  }
  auto fetch = [&](int64_t t) {
    const int64_t rb = t * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t rr = rb + r * RPW;
      rawx[r] = u32x4{0, 0, 0, 0};
      rawd[r] = u32x4{0, 0, 0, 0};
      const bool table = ROPE == 1 || (ROPE == 2 && r == 0);   // as in the forward kernel
      const int f = ROPE == 1 ? r : 0;
      if (table) {
#pragma unroll
        for (int j = 0; j < 8; ++j) fr[f][j] = 0.f;
      }
      if (rr < S && act) {
        const size_t off = (size_t)((b * S + rr) * C + col);
        rawx[r] = load_stream(a.x, off);
        rawd[r] = load_stream(a.dy, off);
        if (table) load_freq8(a.freqs, (size_t)(rp[f].pos * a.head_dim + col), fr[f]);
      }
      if (table) rp[f].advance(a.rows_per_pos, a.seq_len);
    }
  };

  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t rbase = tile * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
    float xf[R][8], df[R][8];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = rbase + r * RPW < S;
      unpack8(rawx[r], xf[r]);
      unpack8(rawd[r], df[r]);
      // the incoming gradient is that of the rotated output: undo the rotation first
      if constexpr (ROPE) rope_unrotate(df[r], fr[ROPE == 1 ? r : 0]);
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);
    if constexpr (NW > 1) __syncthreads();   // lock-step only: keeps the request stream narrow (+1-2 %)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float mean = 0.f;
      if constexpr (ADALN) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) t += xf[r][j];
        mean = group_allsum<L>(t) * a.inv_cols;
      }
      float sv = 0.f, sh_ = 0.f, sg = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float d = xf[r][j];
        if constexpr (ADALN) {
          d -= mean;
          if constexpr (!FULL) d = act ? d : 0.f;
          xf[r][j] = d;
        }
        const float gg = df[r][j] * g[j];
        sv = fmaf(d, d, sv);
        sh_ = fmaf(gg, d, sh_);
        if constexpr (ADALN) sg += gg;
      }
      sv = group_allsum<L>(sv);
      sh_ = group_allsum<L>(sh_);
      if constexpr (ADALN) sg = group_allsum<L>(sg);
      const float rstd = rv[r] ? rsqrtf(sv * a.inv_cols + a.eps) : 0.f;   // padding rows: see the wide kernel
      const float k2 = -(rstd * rstd) * (sh_ * a.inv_cols);
      const float k1 = ADALN ? -rstd * (sg * a.inv_cols) : 0.f;
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float xh = xf[r][j] * rstd;
        const float dyv = df[r][j];
        acc0[j] = fmaf(dyv, xh, acc0[j]);
        if constexpr (ADALN) acc1[j] += dyv;
        o[j] = fmaf(xh, k2, fmaf(dyv * g[j], rstd, k1));
      }
      if (rv[r] && act) store_stream(a.dx, (size_t)((b * S + rbase + r * RPW) * C + col), pack8(o));
    }
  }

  narrow_write_partials<ADALN, L, NW>(acc0, acc1, a.partials, b, C, pi, ri, wave);
}


// ============================================================================ backward from saved tensors
// The reference's contract: backward receives the tensor saved by forward (AdaLN: x_norm,
// RMSNorm: the forward output y, from which x_hat = y / weight) and the per-row rstd,
// instead of x.  Same skeleton as above without the statistics phases.
struct BwdSavedArgs {
  void* dx;
  const void* dy;
  const void* xs;      // AdaLN: x_norm [rows, cols];  RMSNorm: forward output y [rows, cols]
  const void* p0;      // AdaLN: scale [B, C];  RMSNorm: weight [C]
  const float* rstd;   // [rows]
  float* partials;
  int64_t rows_per_batch;
  int64_t n_tiles;
  int cols;
  int packs;
  float inv_cols;
};

template <int KIND, int W, int P, int R, int Q, bool FULL>
__global__ __launch_bounds__(64 * W * Q) void norm_bwd_saved_wide(const BwdSavedArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
  constexpr int NV = ADALN ? 2 : 1;
  __shared__ float red[2][Q][W * R * NV];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = wave / W;
  const int w = wave - q * W;
  const int64_t b = blockIdx.y;
  const int64_t S = a.rows_per_batch;
  const int C = a.cols;

  int col[P];
  bool act[P];
  float g[P][8];    // 1 + scale, or weight
  float gi[P][8];   // RMSNorm: 1 / weight (x_hat = y / weight); 0 on masked lanes
  float acc0[P][8], acc1[P][8];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int pk = p * 64 * W + w * 64 + lane;
    act[p] = FULL || pk < a.packs;
    col[p] = pk * kPack;
    u32x4 r0 = {0, 0, 0, 0};
    if (act[p]) r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col[p]);
    unpack8(r0, g[p]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (ADALN) g[p][j] += 1.0f;
      gi[p][j] = (!ADALN && act[p]) ? 1.0f / g[p][j] : 0.f;
      acc0[p][j] = 0.f;
      acc1[p][j] = 0.f;
    }
  }

  u32x4 rawx[R][P], rawd[R][P];
  float rs[R];
  auto fetch = [&](int64_t t) {
    const int64_t r0 = t * (Q * R) + q * R;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const bool ok = r0 + r < S;
      rs[r] = ok ? a.rstd[b * S + r0 + r] : 0.f;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        rawx[r][p] = u32x4{0, 0, 0, 0};
        rawd[r][p] = u32x4{0, 0, 0, 0};
        if (ok && act[p]) {
          const size_t off = (size_t)((b * S + r0 + r) * C + col[p]);
          rawx[r][p] = load_stream(a.xs, off);
          rawd[r][p] = load_stream(a.dy, off);
        }
      }
    }
  };

  unsigned phase = 0;
  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * (Q * R) + q * R;
    float xh[R][P][8], df[R][P][8], rstd[R];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = row0 + r < S;
      rstd[r] = rs[r];
#pragma unroll
      for (int p = 0; p < P; ++p) {
        unpack8(rawx[r][p], xh[r][p]);
        unpack8(rawd[r][p], df[r][p]);
      }
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);

    float red_v[R * NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s1 = 0.f, s0 = 0.f;
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if constexpr (!ADALN) xh[r][p][j] *= gi[p][j];
          const float gg = df[r][p][j] * g[p][j];
          s1 = fmaf(gg, xh[r][p][j], s1);
          if constexpr (ADALN) s0 += gg;
        }
      red_v[r * NV + 0] = s1;
      if constexpr (ADALN) red_v[r * NV + 1] = s0;
    }
    rowgroup_allsum<W, R * NV>(red_v, red[phase & 1][q], w, lane);
    ++phase;

#pragma unroll
    for (int r = 0; r < R; ++r) {
      // dx = rstd * (g - mean(g) - x_hat * mean(g * x_hat))
      const float k2 = -rstd[r] * (red_v[r * NV + 0] * a.inv_cols);
      const float k1 = ADALN ? -rstd[r] * (red_v[r * NV + 1] * a.inv_cols) : 0.f;
      const int64_t row = b * S + row0 + r;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float dyv = df[r][p][j];
          acc0[p][j] = fmaf(dyv, xh[r][p][j], acc0[p][j]);
          if constexpr (ADALN) acc1[p][j] += dyv;
          o[j] = fmaf(xh[r][p][j], k2, fmaf(dyv * g[p][j], rstd[r], k1));
        }
        if (rv[r] && act[p]) store_stream(a.dx, (size_t)(row * C + col[p]), pack8(o));
      }
    }
  }
  wide_write_partials<ADALN, W, P, Q>(acc0, acc1, act, col, a.partials, b, C, q, w, lane);
}

template <int KIND, int L, int R, int NW, bool FULL>
__global__ __launch_bounds__(64 * NW) void norm_bwd_saved_narrow(const BwdSavedArgs a) {
  constexpr bool ADALN = (KIND == kAdaLN);
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

  float g[8], gi[8], acc0[8], acc1[8];
  {
    u32x4 r0 = {0, 0, 0, 0};
    if (act) r0 = load_cached(a.p0, (ADALN ? b * C : 0) + col);
    unpack8(r0, g);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (ADALN) g[j] += 1.0f;
      gi[j] = (!ADALN && act) ? 1.0f / g[j] : 0.f;
      acc0[j] = 0.f;
      acc1[j] = 0.f;
    }
  }

  u32x4 rawx[R], rawd[R];
  float rs[R];
  auto fetch = [&](int64_t t) {
    const int64_t rb = t * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t rr = rb + r * RPW;
      rawx[r] = u32x4{0, 0, 0, 0};
      rawd[r] = u32x4{0, 0, 0, 0};
      rs[r] = rr < S ? a.rstd[b * S + rr] : 0.f;
      if (rr < S && act) {
        const size_t off = (size_t)((b * S + rr) * C + col);
        rawx[r] = load_stream(a.xs, off);
        rawd[r] = load_stream(a.dy, off);
      }
    }
  };

  int64_t tile = blockIdx.x;
  if (PF && tile < a.n_tiles) fetch(tile);
  for (; tile < a.n_tiles; tile += gridDim.x) {
    const int64_t rbase = tile * (NW * R * RPW) + (int64_t)wave * (R * RPW) + ri;
    float xh[R][8], df[R][8], rstd[R];
    bool rv[R];
    if (!PF) fetch(tile);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      rv[r] = rbase + r * RPW < S;
      rstd[r] = rs[r];
      unpack8(rawx[r], xh[r]);
      unpack8(rawd[r], df[r]);
    }
    if (PF && tile + gridDim.x < a.n_tiles) fetch(tile + gridDim.x);
    if constexpr (NW > 1) __syncthreads();   // lock-step only: keeps the request stream narrow (+1-2 %)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s1 = 0.f, s0 = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if constexpr (!ADALN) xh[r][j] *= gi[j];
        const float gg = df[r][j] * g[j];
        s1 = fmaf(gg, xh[r][j], s1);
        if constexpr (ADALN) s0 += gg;
      }
      s1 = group_allsum<L>(s1);
      if constexpr (ADALN) s0 = group_allsum<L>(s0);
      const float k2 = -rstd[r] * (s1 * a.inv_cols);
      const float k1 = ADALN ? -rstd[r] * (s0 * a.inv_cols) : 0.f;
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float dyv = df[r][j];
        acc0[j] = fmaf(dyv, xh[r][j], acc0[j]);
        if constexpr (ADALN) acc1[j] += dyv;
        o[j] = fmaf(xh[r][j], k2, fmaf(dyv * g[j], rstd[r], k1));
      }
      if (rv[r] && act) store_stream(a.dx, (size_t)((b * S + rbase + r * RPW) * C + col), pack8(o));
    }
  }
  narrow_write_partials<ADALN, L, NW>(acc0, acc1, a.partials, b, C, pi, ri, wave);
}

// ============================================================================ second pass
// out[acc][b][c] = sum_j partials[b][j][acc][c], j in a fixed order: 16 waves take
// the partials j = wave, wave+16, ... and are then folded in wave order through LDS.
// The output is fp32, or bf16 (rounded once) when out_bf16 is set.
template <int NACC>
__global__ __launch_bounds__(1024) void reduce_partials(void* __restrict__ out0, void* __restrict__ out1,
                                                        void* __restrict__ out2, const float* __restrict__ partials,
                                                        int n_partials, int cols, int out_bf16) {
  __shared__ float fold[16][NACC][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int64_t b = blockIdx.y;
  float s[NACC];
#pragma unroll
  for (int acc = 0; acc < NACC; ++acc) s[acc] = 0.f;
  if (c < cols) {
    const float* base = partials + (size_t)b * n_partials * NACC * cols + c;
    // 8 independent loads per accumulator in flight, in the ragged last round too (a missing
    // partial contributes +0.0f, which changes no sum); the sum order stays fixed.
    for (int j = wave; j < n_partials; j += 8 * 16) {
      float t[8][NACC];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int acc = 0; acc < NACC; ++acc)
          t[u][acc] = j + u * 16 < n_partials ? base[((size_t)(j + u * 16) * NACC + acc) * cols] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int acc = 0; acc < NACC; ++acc) s[acc] += t[u][acc];
    }
  }
#pragma unroll
  for (int acc = 0; acc < NACC; ++acc) fold[wave][acc][lane] = s[acc];
  __syncthreads();
  if (wave < NACC && c < cols) {
    float t = fold[0][wave][lane];
#pragma unroll
    for (int ww = 1; ww < 16; ++ww) t += fold[ww][wave][lane];
    void* out = wave == 0 ? out0 : wave == 1 ? out1 : out2;
    const size_t idx = (size_t)b * cols + c;
    if (out_bf16) static_cast<uint16_t*>(out)[idx] = f32_to_bf16(t);
    else          static_cast<float*>(out)[idx] = t;
  }
}

}  // namespace tt
