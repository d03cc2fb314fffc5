// Shared device helpers for the gfx950 fused-normalisation kernels:
// 128-bit bf16 pack load/store, bf16<->fp32 conversion, wave64 DPP reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tt {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;   // CDNA wavefront width
constexpr int kPack = 8;    // bf16 elements per 128-bit pack

// ---------------------------------------------------------------- memory
// Streaming tensors are touched exactly once, so they bypass cache retention: "nt" global
// loads, and stores with system scope on top ("sc0 sc1 nt": written through instead of being
// kept in L2), which measured 1-2 % faster than plain "nt" stores under the 2-reads-1-write mix
// of the backward kernels.  The compiler's builtin only offers "nt", hence the asm for stores;
// it is an ordinary vector store.  Parameters use ordinary cached loads.
__device__ __forceinline__ u32x4 load_stream(const void* base, size_t elem_off) {
  const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + elem_off);
  return __builtin_nontemporal_load(p);
}
__device__ __forceinline__ void store_stream(void* base, size_t elem_off, u32x4 v) {
  u32x4* p = reinterpret_cast<u32x4*>(static_cast<uint16_t*>(base) + elem_off);
  // The compiler pads its own stores wider than 64 bits against two hazards of this target but
  // cannot see inside the asm, so the padding is spelled out: two wait states between a VALU
  // write of the data registers and the store, and two between the store and the next VALU
  // write of those registers (the data is read after issue).  Four are spent on each side.
  asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
}
// Two stores of one lane to the same element offset of two tensors (an output and a second
// saved copy): one asm block, so the pair pays the hazard padding once.
__device__ __forceinline__ void store_stream2(void* base0, void* base1, size_t elem_off, u32x4 v0, u32x4 v1) {
  u32x4* p0 = reinterpret_cast<u32x4*>(static_cast<uint16_t*>(base0) + elem_off);
  u32x4* p1 = reinterpret_cast<u32x4*>(static_cast<uint16_t*>(base1) + elem_off);
  asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %2, off sc0 sc1 nt\n\t"
               "global_store_dwordx4 %1, %3, off sc0 sc1 nt\n\ts_nop 3" ::"v"(p0), "v"(p1), "v"(v0), "v"(v1) : "memory");
}
__device__ __forceinline__ u32x4 load_cached(const void* base, size_t elem_off) {
  return *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + elem_off);
}

// ---------------------------------------------------------------- bf16 <-> fp32
__device__ __forceinline__ void unpack8(u32x4 raw, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j]     = __builtin_bit_cast(float, raw[j] << 16);
    f[2 * j + 1] = __builtin_bit_cast(float, raw[j] & 0xffff0000u);
  }
}
// Round-to-nearest-even fp32 -> bf16, two at a time (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ unsigned pack2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(unsigned, r);
}
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
  u32x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = pack2(f[2 * j], f[2 * j + 1]);
  return o;
}
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, static_cast<unsigned>(h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return static_cast<uint16_t>(pack2(f, 0.f) & 0xffffu);
}

// ---------------------------------------------------------------- wave64 reductions
// DPP controls: quad_perm[1,0,3,2]=0xB1, quad_perm[2,3,0,1]=0x4E,
// row_half_mirror=0x141, row_mirror=0x140.  Each step adds a lane's partner, so
// after k steps every lane of an aligned 2^k group holds that group's sum.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, t);
}
__device__ __forceinline__ float readlane(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over aligned groups of L lanes (L in 1,2,4,8,16,32,64); every lane of a
// group receives the group's total.  The summation order is fixed, so results
// are bitwise reproducible.
template <int L>
__device__ __forceinline__ float group_allsum(float v) {
  if constexpr (L >= 2) v = dpp_add<0xB1>(v);
  if constexpr (L >= 4) v = dpp_add<0x4E>(v);
  if constexpr (L >= 8) v = dpp_add<0x141>(v);
  if constexpr (L >= 16) v = dpp_add<0x140>(v);
  if constexpr (L == 32) {
    // partner row inside the 32-lane half: lane ^ 16
    int t = __builtin_amdgcn_ds_bpermute(((int)(threadIdx.x & 63) ^ 16) << 2, __builtin_bit_cast(int, v));
    v += __builtin_bit_cast(float, t);
  }
  if constexpr (L == 64) {
    float a = readlane(v, 0), b = readlane(v, 16), c = readlane(v, 32), d = readlane(v, 48);
    v = (a + b) + (c + d);
  }
  return v;
}
__device__ __forceinline__ float wave_allsum(float v) { return group_allsum<64>(v); }

}  // namespace tt
