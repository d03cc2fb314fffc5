// Table of compiled kernel variants and the host-side lookup that maps a row
// width to one of them.  Each of the four kernel families (AdaLN / RMSNorm x
// forward / backward) is instantiated in its own translation unit through the
// lookup templates below, so the families compile in parallel.
#pragma once
#include "gate_kernels.hpp"
#include "norm_kernels.hpp"
#include "resnorm_kernels.hpp"

namespace tt {

struct KernelInfo {
  const void* fn;   // __global__ function taking one FwdArgs / BwdArgs by value
  int threads;      // workgroup size
  int tile_rows;    // rows one workgroup consumes per loop iteration
  int lane_loads;   // 128-bit loads per lane and streamed tensor in one tile
};

// Wide variants: (index, W waves per row, P packs per lane).  A row of `packs`
// 128-bit packs runs on the variant with the fewest lane slots 64*W*P >= packs.
#define TT_WIDE_LIST(X) \
  X(0, 1, 1) X(1, 2, 1) X(2, 3, 1) X(3, 4, 1) X(4, 3, 2) X(5, 4, 2) X(6, 5, 2) \
  X(7, 6, 2) X(8, 8, 2) X(9, 12, 2) X(10, 16, 2) X(11, 16, 4)
constexpr int kNumWide = 12;
constexpr int kWideW[kNumWide] = {1, 2, 3, 4, 3, 4, 5, 6, 8, 12, 16, 16};
constexpr int kWideP[kNumWide] = {1, 1, 1, 1, 2, 2, 2, 2, 2, 2, 2, 4};

// Narrow variants: (index, L lanes per row).
#define TT_NARROW_LIST(X) X(0, 1) X(1, 2) X(2, 4) X(3, 8) X(4, 16) X(5, 32)
constexpr int kNumNarrow = 6;
constexpr int kNarrowL[kNumNarrow] = {1, 2, 4, 8, 16, 32};
constexpr int kNarrowMaxPacks = 32;
constexpr int kMaxPacks = 64 * 16 * 4;

// ---- tuning constants, from sweeps on MI355X (see make_plan in capi.hip for the grid rule)
// R: rows in flight per row group;  Q: row groups per workgroup.  HBM throughput peaks with
// roughly 18 (forward) / 12 (backward, two input tensors) outstanding 128-bit loads per lane
// column of a CU and tensor, and barrier-coupled row groups in ONE workgroup per CU stream
// better than independent workgroups; Q is chosen so that one workgroup carries that load.
constexpr int kNarrowR = 2;    // loads per lane and tensor in flight, narrow kernels
// RMSNorm backward on narrow rows streams better with six loads per lane in ONE four-wave workgroup
// per CU than with two loads in two workgroups: 2,851,200 x 128 backward 362 -> 354 us between
// forward launches (reference contract 371 -> 358 us), 1-1.5 % at 32, 64 and 256 columns.  Forward
// and the AdaLN kernels lose with six (128 columns forward 242 -> 269 us, AdaLN backward 359 -> 363 us).
constexpr int kNarrowRmsBwdR = 6;
// RMSNorm forward on narrow rows with every lane slot in use: six loads per lane as well.  As fast as
// two (2,851,200 x 128: 242 us either way; 16 ... 256 columns within 1 %), but with two the time depends
// on where the output lies relative to the input (period 128 MiB: 243 us over three quarters of it,
// up to 279 us over the rest), with six it does not (240-244 us at every offset).  Masked widths keep
// two (96 columns 282 -> 285 us, 200 columns 369 -> 382 us with six).
constexpr int kNarrowRmsFwdFullR = 6;
constexpr int kNarrowNW = 4;   // independent waves per workgroup, narrow kernels
constexpr int kFwdLoadsPerCu = 18;   // target waves x loads-per-lane per CU, forward
constexpr int kBwdLoadsPerCu = 12;   // same, backward (per input tensor)
constexpr int kFwdXnLoadsPerCu = 12; // same, AdaLN forward that also stores x_norm (see fwd_xn_wide_Q)

constexpr int fwd_wide_R(int W, int P) { return 1; }   // two rows per tile: 1-3 % slower at every width
constexpr int bwd_wide_R(int W, int P) { return 1; }
// AdaLN backward has two barrier-coupled reductions per row; on the variants below two rows per
// row group and tile (both rows share each exchange) hide that latency better.  Measured,
// us at R = 1 -> R = 2: 32760 x 1536: 53.8 -> 51.9; 4 x 32760 x 1536: 200.8 -> 198.0;
// 150000 x 2048: 300.9 -> 290.0; 118800 x 3072: 358.4 -> 348.9; 60000 x 6144: 381.2 -> 355.4;
// 300000 x 1024: 290.7 -> 288.5.  Worse with R = 2: 512 columns (156.9 -> 169.0), 4096
// (356.6 -> 368.8), 8192 (358.0 -> 399.5), and 5120 (ten waves: spills).  RMSNorm (one reduction
// per row) is 2-3 % slower with R = 2 everywhere.
constexpr int adaln_bwd_wide_R(int W, int P) {
  return ((P == 1 && W >= 2 && W <= 4) || (P == 2 && (W == 3 || W == 6))) ? 2 : bwd_wide_R(W, P);
}
constexpr int fwd_wide_Q(int W, int P) {
  return W >= 7 ? 1 : (10 + W / 2) / W;          // about 10 waves per workgroup
}
constexpr int bwd_wide_Q(int W, int P) {
  int q = (2 * kBwdLoadsPerCu + W * P) / (2 * W * P);   // round(12 / (W*P))
  if (q < 1) q = 1;
  if (W * q < 6) q = (6 + W - 1) / W;                   // at least 6 waves to keep up with the arithmetic
  while (q > 1 && W * q > 12) --q;                      // at most 12 waves: 170 VGPRs per lane
  return q;
}

// Index of the wide variant for `packs` (> kNarrowMaxPacks), or -1.
inline int select_wide(int packs) {
  int best = -1, best_slots = 1 << 30;
  for (int i = 0; i < kNumWide; ++i) {
    const int slots = 64 * kWideW[i] * kWideP[i];
    // fewest slots wins; on a tie the later entry (more packs per lane, fewer waves) wins
    if (slots >= packs && slots <= best_slots) { best = i; best_slots = slots; }
  }
  return best;
}
inline int select_narrow(int packs) {
  for (int i = 0; i < kNumNarrow; ++i)
    if (kNarrowL[i] >= packs) return i;
  return -1;
}

template <int KIND, int W, int P, bool FULL>
KernelInfo info_fwd_wide() {
  constexpr int R = fwd_wide_R(W, P), Q = fwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_fwd_wide<KIND, W, P, R, Q, FULL>), 64 * W * Q, Q * R, P * R};
}
template <int KIND, int W, int P, bool FULL>
KernelInfo info_bwd_wide() {
  constexpr int R = KIND == kAdaLN ? adaln_bwd_wide_R(W, P) : bwd_wide_R(W, P), Q = bwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_bwd_wide<KIND, W, P, R, Q, FULL>), 64 * W * Q, Q * R, P * R};
}
template <int KIND, int W, int P, bool FULL>
KernelInfo info_bwd_saved_wide() {
  constexpr int R = bwd_wide_R(W, P), Q = bwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_bwd_saved_wide<KIND, W, P, R, Q, FULL>), 64 * W * Q, Q * R, P * R};
}
template <int KIND, int L, bool FULL>
KernelInfo info_bwd_saved_narrow() {
  constexpr int R = KIND == kRMS ? kNarrowRmsBwdR : kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_bwd_saved_narrow<KIND, L, R, NW, FULL>), 64 * NW, NW * R * (64 / L), R};
}
template <int KIND, int L, bool FULL>
KernelInfo info_fwd_narrow() {
  constexpr int R = (KIND == kRMS && FULL) ? kNarrowRmsFwdFullR : kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_fwd_narrow<KIND, L, R, NW, FULL>), 64 * NW, NW * R * (64 / L), R};
}
template <int KIND, int L, bool FULL>
KernelInfo info_bwd_narrow() {
  constexpr int R = KIND == kRMS ? kNarrowRmsBwdR : kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_bwd_narrow<KIND, L, R, NW, FULL>), 64 * NW, NW * R * (64 / L), R};
}

// AdaLN forward that also stores x_norm (the reference's forward contract): one read and two
// write streams.  Bare streams of that mix (no arithmetic) reach 5.7-5.9 TB/s on MI355X (370-385 us
// for the 2.19 GB of 118800 x 3072), and like writes on their own they go fastest with FEW requests
// in flight: about 12 loads per lane column of a CU (kFwdXnLoadsPerCu), not the 18-20 of the
// one-output forward.  One row group per workgroup and several independent workgroups per CU:
// barrier-coupled row groups are 1 % faster at best (118800 x 3072: 379-383 us against 384-390) but
// 5-8 % slower (400-413 us) over a quarter of the possible placements of the two outputs relative to
// the input (period 128 MiB); independent workgroups stay at 384-393 us at every placement.
// Measured with this rule: 75600 x 5120 416 us, 131040 x 1536 213 us, 150000 x 2048 323 us.
constexpr int fwd_xn_wide_Q(int W, int P) { return 1; }
template <int W, int P, bool FULL>
KernelInfo info_fwd_xn_wide() {
  constexpr int R = fwd_wide_R(W, P), Q = fwd_xn_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_fwd_wide<kAdaLN, W, P, R, Q, FULL, false, true>), 64 * W * Q, Q * R, P * R};
}
template <int L, bool FULL>
KernelInfo info_fwd_xn_narrow() {
  constexpr int R = kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_fwd_narrow<kAdaLN, L, R, NW, FULL, 0, true>), 64 * NW, NW * R * (64 / L), R};
}
inline KernelInfo lookup_fwd_xn(bool narrow, int idx, bool full) {
  if (narrow) {
    switch (idx) {
#define X(i, L) case i: return full ? info_fwd_xn_narrow<L, true>() : info_fwd_xn_narrow<L, false>();
      TT_NARROW_LIST(X)
#undef X
    }
  } else {
    switch (idx) {
#define X(i, W, P) case i: return full ? info_fwd_xn_wide<W, P, true>() : info_fwd_xn_wide<W, P, false>();
      TT_WIDE_LIST(X)
#undef X
    }
  }
  return {nullptr, 0, 0, 0};
}

template <int KIND>
KernelInfo lookup_fwd(bool narrow, int idx, bool full) {
  if (narrow) {
    switch (idx) {
#define X(i, L) case i: return full ? info_fwd_narrow<KIND, L, true>() : info_fwd_narrow<KIND, L, false>();
      TT_NARROW_LIST(X)
#undef X
    }
  } else {
    switch (idx) {
#define X(i, W, P) case i: return full ? info_fwd_wide<KIND, W, P, true>() : info_fwd_wide<KIND, W, P, false>();
      TT_WIDE_LIST(X)
#undef X
    }
  }
  return {nullptr, 0, 0, 0};
}
template <int KIND>
KernelInfo lookup_bwd(bool narrow, int idx, bool full) {
  if (narrow) {
    switch (idx) {
#define X(i, L) case i: return full ? info_bwd_narrow<KIND, L, true>() : info_bwd_narrow<KIND, L, false>();
      TT_NARROW_LIST(X)
#undef X
    }
  } else {
    switch (idx) {
#define X(i, W, P) case i: return full ? info_bwd_wide<KIND, W, P, true>() : info_bwd_wide<KIND, W, P, false>();
      TT_WIDE_LIST(X)
#undef X
    }
  }
  return {nullptr, 0, 0, 0};
}

// RMSNorm with the rotary embedding fused behind it (wide rows only).
template <int W, int P, bool FULL>
KernelInfo info_fwd_rope_wide() {
  constexpr int R = fwd_wide_R(W, P), Q = fwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_fwd_wide<kRMS, W, P, R, Q, FULL, true>), 64 * W * Q, Q * R, P * R};
}
template <int W, int P, bool FULL>
KernelInfo info_bwd_rope_wide() {
  constexpr int R = bwd_wide_R(W, P), Q = bwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&norm_bwd_wide<kRMS, W, P, R, Q, FULL, true>), 64 * W * Q, Q * R, P * R};
}
template <int L, bool FULL>
KernelInfo info_fwd_rope_narrow() {
  constexpr int R = kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_fwd_narrow<kRMS, L, R, NW, FULL, true>), 64 * NW, NW * R * (64 / L), R};
}
template <int L, bool FULL>
KernelInfo info_bwd_rope_narrow() {
  constexpr int R = kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&norm_bwd_narrow<kRMS, L, R, NW, FULL, true>), 64 * NW, NW * R * (64 / L), R};
}
// Token mode of the narrow ROPE kernels (ROPE = 2: the rows a wave takes per tile are the heads of
// one token, so the (cos, sin) entries are loaded once per tile and lane).  Instantiated for rows of
// 16 lanes (head_dim 72 ... 128) and 24 heads per token, HunyuanVideo's layout: 24 rows / 4 rows per
// load = 6 loads per lane.
constexpr int kRopeTokenL = 16, kRopeTokenR = 6, kRopeTokenHeads = kRopeTokenR * (64 / kRopeTokenL);
// Four waves in one workgroup per CU (24 loads per lane column and tensor in flight) measured best:
// forward 245 us, backward + reduction 356 us at 118800 x 24 x 128; 5 / 6 / 8 waves: 277 / 265 / 267 us
// forward, 378 / 368 / 380 us backward; 2 and 3 waves need 2-3 workgroups per CU and reach 259-265 us.
constexpr int kRopeTokenNW = 4;
template <bool FULL>
KernelInfo info_rope_token(bool backward) {
  constexpr int L = kRopeTokenL, R = kRopeTokenR, NF = kRopeTokenNW, NB = kRopeTokenNW;
  if (backward)
    return {reinterpret_cast<const void*>(&norm_bwd_narrow<kRMS, L, R, NB, FULL, 2>), 64 * NB, NB * R * (64 / L), R};
  return {reinterpret_cast<const void*>(&norm_fwd_narrow<kRMS, L, R, NF, FULL, 2>), 64 * NF, NF * R * (64 / L), R};
}
inline KernelInfo lookup_rope(bool narrow, bool backward, int idx, bool full, int64_t heads) {
  if (narrow && kNarrowL[idx] == kRopeTokenL && heads == kRopeTokenHeads)
    return full ? info_rope_token<true>(backward) : info_rope_token<false>(backward);
  if (narrow) {
    switch (idx) {
#define X(i, L)                                                                                       \
  case i:                                                                                             \
    return backward ? (full ? info_bwd_rope_narrow<L, true>() : info_bwd_rope_narrow<L, false>())     \
                    : (full ? info_fwd_rope_narrow<L, true>() : info_fwd_rope_narrow<L, false>());
      TT_NARROW_LIST(X)
#undef X
    }
    return {nullptr, 0, 0, 0};
  }
  switch (idx) {
#define X(i, W, P)                                                                                  \
  case i:                                                                                           \
    return backward ? (full ? info_bwd_rope_wide<W, P, true>() : info_bwd_rope_wide<W, P, false>()) \
                    : (full ? info_fwd_rope_wide<W, P, true>() : info_fwd_rope_wide<W, P, false>());
    TT_WIDE_LIST(X)
#undef X
  }
  return {nullptr, 0, 0, 0};
}

template <int MODE, int W, int P, bool FULL>
KernelInfo info_gate_wide() {
  constexpr int R = bwd_wide_R(W, P), Q = bwd_wide_Q(W, P);
  return {reinterpret_cast<const void*>(&gate_wide<MODE, W, P, R, Q, FULL>), 64 * W * Q, Q * R, P * R};
}
template <int MODE, int L, bool FULL>
KernelInfo info_gate_narrow() {
  constexpr int R = kNarrowR, NW = kNarrowNW;
  return {reinterpret_cast<const void*>(&gate_narrow<MODE, L, R, NW, FULL>), 64 * NW, NW * R * (64 / L), R};
}
template <int MODE>
KernelInfo lookup_gate(bool narrow, int idx, bool full) {
  if (narrow) {
    switch (idx) {
#define X(i, L) case i: return full ? info_gate_narrow<MODE, L, true>() : info_gate_narrow<MODE, L, false>();
      TT_NARROW_LIST(X)
#undef X
    }
  } else {
    switch (idx) {
#define X(i, W, P) case i: return full ? info_gate_wide<MODE, W, P, true>() : info_gate_wide<MODE, W, P, false>();
      TT_WIDE_LIST(X)
#undef X
    }
  }
  return {nullptr, 0, 0, 0};
}

// Residual update fused with the following LayerNorm (wide rows only): forward streams two
// inputs, backward three (four with a gate).
// Row groups per workgroup for the kernels with two to four streamed inputs, from sweeps on
// MI355X: about ten waves where a lane holds one pack per tensor; with two packs per lane as many
// row groups as fit in eight waves, which leaves the backward kernels their 170-235 VGPRs
// (ten waves cap them at 168 and they spill).  Measured (forward / backward / gated backward, us):
// 1536 columns 281 / 271 / 418 with 9 waves against 302 / 287 / 459 with 3; 2048: 207 / 203 / 326
// with 12 waves against 221 / 212 / 362 with 4; 3072 x 118800 rows: 492 / 477 / 746 with 6 waves;
// 4096 x 90000: 502 / 478 / 763 with 8 waves against 522 / 523 / 888 with 4; 5120: 519 / 525 / 786
// with 5 waves against 533 / 595 / 2437 with 10.
constexpr int res_waves_Q(int W, int P) {
  const int q = P == 1 ? (10 + W / 2) / W : 8 / W;
  return q < 1 ? 1 : q;
}
constexpr int res_fwd_Q(int W, int P) {
  return res_waves_Q(W, P);
}
constexpr int res_bwd_Q(int W, int P, bool gated) {
  return res_waves_Q(W, P);
}
template <int W, int P, bool FULL, bool GATED>
KernelInfo info_res_fwd() {
  constexpr int R = 1, Q = res_fwd_Q(W, P);
  return {reinterpret_cast<const void*>(&resnorm_fwd_wide<W, P, R, Q, FULL, GATED>), 64 * W * Q, Q * R, P * R};
}
template <int W, int P, bool FULL, bool GATED>
KernelInfo info_res_bwd() {
  constexpr int R = 1, Q = res_bwd_Q(W, P, GATED);
  return {reinterpret_cast<const void*>(&resnorm_bwd_wide<W, P, R, Q, FULL, GATED>), 64 * W * Q, Q * R, P * R};
}
template <bool GATED>
KernelInfo lookup_res(bool backward, int idx, bool full) {
  switch (idx) {
#define X(i, W, P)                                                                                        \
  case i:                                                                                                 \
    return backward ? (full ? info_res_bwd<W, P, true, GATED>() : info_res_bwd<W, P, false, GATED>())     \
                    : (full ? info_res_fwd<W, P, true, GATED>() : info_res_fwd<W, P, false, GATED>());
    TT_WIDE_LIST(X)
#undef X
  }
  return {nullptr, 0, 0, 0};
}

template <int KIND>
KernelInfo lookup_bwd_saved(bool narrow, int idx, bool full) {
  if (narrow) {
    switch (idx) {
#define X(i, L) case i: return full ? info_bwd_saved_narrow<KIND, L, true>() : info_bwd_saved_narrow<KIND, L, false>();
      TT_NARROW_LIST(X)
#undef X
    }
  } else {
    switch (idx) {
#define X(i, W, P) case i: return full ? info_bwd_saved_wide<KIND, W, P, true>() : info_bwd_saved_wide<KIND, W, P, false>();
      TT_WIDE_LIST(X)
#undef X
    }
  }
  return {nullptr, 0, 0, 0};
}

// Defined one per translation unit (adaln_fwd.hip, adaln_fwd_xnorm.hip, adaln_bwd.hip, adaln_bwd_saved.hip, rms_fwd.hip, rms_bwd.hip, rms_bwd_saved.hip, rms_rope.hip, gate.hip,
// resnorm_plain.hip, resnorm_gated.hip).
KernelInfo adaln_fwd_kernel(bool narrow, int idx, bool full);
KernelInfo adaln_fwd_xnorm_kernel(bool narrow, int idx, bool full);
KernelInfo adaln_bwd_kernel(bool narrow, int idx, bool full);
KernelInfo rms_fwd_kernel(bool narrow, int idx, bool full);
KernelInfo rms_bwd_kernel(bool narrow, int idx, bool full);
KernelInfo adaln_bwd_saved_kernel(bool narrow, int idx, bool full);
KernelInfo rms_bwd_saved_kernel(bool narrow, int idx, bool full);
KernelInfo rms_rope_kernel(bool narrow, bool backward, int idx, bool full, int64_t heads);
KernelInfo gate_fwd_kernel(bool narrow, int idx, bool full);
KernelInfo gate_bwd_kernel(bool narrow, int idx, bool full);
KernelInfo resnorm_plain_kernel(bool backward, int idx, bool full);
KernelInfo resnorm_gated_kernel(bool backward, int idx, bool full);

}  // namespace tt
