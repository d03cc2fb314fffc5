// Stand-alone measurement program (no part of the library): what do bare HBM streams reach on the
// GPU at hand, and does any way of issuing the stores lift the mixed read+write ceiling?
//
// Streams n = 75600 x 640 packs of 16 bytes (the headline tensor, 774,144,000 bytes) with no
// arithmetic in four traffic mixes (write only, read only, 1 read : 1 write, 2 reads : 1 write) under
//   addr   the address layout: "strided" (pack = it*G*T*U + u*G*T + g*T + t: what the normalisation
//          kernels do, tile by tile), "chunk" (each workgroup a contiguous T*U-pack chunk per
//          iteration), "slab" (each workgroup one contiguous share of the tensor), "pairs" (a lane
//          owns two adjacent packs: 32 contiguous bytes per lane and store pair)
//   store  how stores are issued: "global" (global_store_dwordx4) with one of four cache policies,
//          "buffer" (buffer_store_dwordx4, same policy bits), "staged" (the tile goes through LDS
//          and ONE wave of the workgroup streams it out, the role rotating from tile to tile)
//   T, G, U  threads per workgroup, workgroups, packs per lane in flight
// Each configuration is timed with HIP events over 9 launches that alternate between two buffer
// sets; the median is printed.  Every variant is checked once against the expected bytes.
// Output: one line per configuration, then the best line per (mix, addr, store).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <map>
#include <string>
#include <vector>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define CK(x)                                                                     \
  do {                                                                            \
    hipError_t err_ = (x);                                                        \
    if (err_ != hipSuccess) {                                                     \
      printf("HIP error %s at line %d\n", hipGetErrorString(err_), __LINE__);     \
      exit(1);                                                                    \
    }                                                                             \
  } while (0)

enum Mix { kWrite = 0, kRead = 1, kCopy = 2, kTwoReads = 3 };
enum Addr { kStrided = 0, kChunk = 1, kSlab = 2, kPairs = 3 };
// store policies: 0 plain, 1 nt, 2 sc0 sc1 nt (the library's), 3 sc1
template <int SP>
__device__ __forceinline__ void store_pack(u32x4* p, u32x4 v) {
  // s_nop: wait states between a VALU write of the data registers and the store, which the
  // compiler cannot insert for an asm statement
  if constexpr (SP == 0) asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %1, off\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
  if constexpr (SP == 1) asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %1, off nt\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
  if constexpr (SP == 2) asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
  if constexpr (SP == 3) asm volatile("s_nop 3\n\tglobal_store_dwordx4 %0, %1, off sc1\n\ts_nop 3" ::"v"(p), "v"(v) : "memory");
}

__device__ __forceinline__ u32x4 index_pattern(size_t i) {
  const unsigned w = (unsigned)i;
  return u32x4{w, w, w, w};
}

// BUF: stores through a raw buffer resource over the whole output (aux 19 = sc0 sc1 nt).
template <int MIX, int ADDR, int U, int SP, bool BUF>
__global__ void __launch_bounds__(1024) flat(const u32x4* __restrict__ a, const u32x4* __restrict__ b, u32x4* __restrict__ c,
                                             size_t n, size_t slab) {
  const size_t G = gridDim.x, T = blockDim.x, g = blockIdx.x, t = threadIdx.x;
  size_t base, step, end;
  if (ADDR == kStrided) { base = g * T + t; step = G * T * U; end = n; }
  else if (ADDR == kSlab) { base = g * slab; step = T * U; end = base + slab < n ? base + slab : n; }
  else { base = g * T * U; step = G * T * U; end = n; }
  __amdgpu_buffer_rsrc_t rc;
  if constexpr (BUF) rc = __builtin_amdgcn_make_buffer_rsrc(c, 0, (int)(n * 16), 0x00020000);
  for (; base < end; base += step) {
    size_t idx[U];
    u32x4 va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ADDR == kStrided) idx[u] = base + u * G * T;
      else if (ADDR == kPairs) idx[u] = base + (u / 2) * 2 * T + 2 * t + (u & 1);
      else idx[u] = base + u * T + t;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      va[u] = index_pattern(idx[u]);
      vb[u] = u32x4{0, 0, 0, 0};
      if (idx[u] < end) {
        if (MIX != kWrite) va[u] = __builtin_nontemporal_load(a + idx[u]);
        if (MIX == kTwoReads) vb[u] = __builtin_nontemporal_load(b + idx[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (MIX == kRead) asm volatile("" ::"v"(va[u]));   // keeps the load and its wait alive
      else if (idx[u] < end) {
        if constexpr (BUF) __builtin_amdgcn_raw_buffer_store_b128(va[u] ^ vb[u], rc, (int)(idx[u] * 16), 0, 19);
        else store_pack<SP>(c + idx[u], va[u] ^ vb[u]);
      }
    }
  }
}

// Tile kernel with the structure of the normalisation kernels: persistent grid, tile += G, the
// next tile prefetched, one barrier per tile.  STAGED = false: every lane stores its own packs.
// STAGED = true: the tile is written to LDS (two buffers) and one wave, rotating from tile to
// tile, streams the whole tile out.
template <int MIX, int NW, int PPT, bool STAGED>
__global__ void __launch_bounds__(64 * NW) tiled(const u32x4* __restrict__ a, const u32x4* __restrict__ b,
                                                 u32x4* __restrict__ c, size_t n_tiles) {
  constexpr int NT = 64 * NW, TP = NT * PPT;
  __shared__ u32x4 lds[STAGED ? 2 * TP : 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  u32x4 ra[PPT], rb[PPT];
  auto fetch = [&](size_t t) {
#pragma unroll
    for (int k = 0; k < PPT; ++k) {
      const size_t i = t * TP + k * NT + tid;
      ra[k] = __builtin_nontemporal_load(a + i);
      if (MIX == kTwoReads) rb[k] = __builtin_nontemporal_load(b + i);
    }
  };
  size_t tile = blockIdx.x, it = 0;
  unsigned par = 0;
  if (tile < n_tiles) fetch(tile);
  for (; tile < n_tiles; tile += gridDim.x, par ^= 1u, ++it) {
    u32x4 v[PPT];
#pragma unroll
    for (int k = 0; k < PPT; ++k) v[k] = MIX == kTwoReads ? (ra[k] ^ rb[k]) : ra[k];
    if (tile + gridDim.x < n_tiles) fetch(tile + gridDim.x);
    if constexpr (!STAGED) {
      __syncthreads();
#pragma unroll
      for (int k = 0; k < PPT; ++k) store_pack<2>(c + tile * TP + k * NT + tid, v[k]);
    } else {
      u32x4* buf = lds + par * TP;
#pragma unroll
      for (int k = 0; k < PPT; ++k) buf[k * NT + tid] = v[k];
      // One barrier per tile is enough: a buffer is rewritten two tiles later, after every wave
      // has passed the next tile's barrier, which the storing wave reaches after its LDS reads.
      __syncthreads();
      if (wave == (int)(it % NW)) {
        constexpr int PER = TP / 64;
#pragma unroll 4
        for (int j = 0; j < PER; ++j) store_pack<2>(c + tile * TP + j * 64 + lane, buf[j * 64 + lane]);
      }
    }
  }
}

// mismatches of c against the expected bytes of a mix over the first n packs
template <int MIX>
__global__ void check(const u32x4* a, const u32x4* b, const u32x4* c, size_t n, unsigned long long* bad) {
  unsigned long long local = 0;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const u32x4 want = MIX == kWrite ? index_pattern(i) : MIX == kCopy ? a[i] : (a[i] ^ b[i]);
    const u32x4 got = c[i];
    local += (got.x != want.x) + (got.y != want.y) + (got.z != want.z) + (got.w != want.w);
  }
  if (local) atomicAdd(bad, local);
}

static u32x4* buf[6];
static unsigned long long* bad;
static const size_t N = (size_t)75600 * 640;
static const char* mix_name[] = {"write", "read", "copy", "2r1w"};
static const double mix_bytes[] = {1.0, 1.0, 2.0, 3.0};
static std::map<std::string, std::pair<double, std::string>> best;
static int failures = 0;

static double median_us(const std::function<void(int)>& launch) {
  const int iters = 9;
  std::vector<hipEvent_t> ev(iters + 1);
  for (auto& e : ev) CK(hipEventCreate(&e));
  for (int w = 0; w < 2; ++w) launch(w & 1);
  CK(hipEventRecord(ev[0]));
  for (int it = 0; it < iters; ++it) {
    launch(it & 1);
    CK(hipEventRecord(ev[it + 1]));
  }
  CK(hipDeviceSynchronize());
  std::vector<float> t(iters);
  for (int it = 0; it < iters; ++it) CK(hipEventElapsedTime(&t[it], ev[it], ev[it + 1]));
  std::sort(t.begin(), t.end());
  for (auto& e : ev) CK(hipEventDestroy(e));
  return t[iters / 2] * 1e3;
}

template <int MIX>
static void verify(const char* what, size_t n) {
  if (MIX == kRead) return;
  CK(hipMemset(bad, 0, 8));
  check<MIX><<<1024, 256>>>(buf[3], buf[4], buf[5], n, bad);   // both buffer sets were written by the timed launches
  unsigned long long h0 = 0, h1 = 0;
  CK(hipMemcpy(&h1, bad, 8, hipMemcpyDeviceToHost));
  CK(hipMemset(bad, 0, 8));
  check<MIX><<<1024, 256>>>(buf[0], buf[1], buf[2], n, bad);
  CK(hipMemcpy(&h0, bad, 8, hipMemcpyDeviceToHost));
  if (h0 || h1) {
    printf("VERIFY FAILED %s: %llu / %llu wrong words\n", what, h0, h1);
    ++failures;
  }
}

static void report(int mix, const char* addr, const char* store, int T, int G, int U, double us, double bytes) {
  const double tbs = bytes / us / 1e6;
  char line[256];
  snprintf(line, sizeof line, "%-5s addr=%-7s store=%-10s T=%4d G=%4d U=%d : %7.1f us %5.2f TB/s", mix_name[mix], addr, store,
           T, G, U, us, tbs);
  puts(line);
  fflush(stdout);
  const std::string key = std::string(mix_name[mix]) + " addr=" + addr + " store=" + store;
  auto it = best.find(key);
  if (it == best.end() || tbs > it->second.first) best[key] = {tbs, line};
}

static const char* addr_name[] = {"strided", "chunk", "slab", "pairs"};
static const char* sp_name[] = {"global", "global-nt", "global-wt", "global-sc1"};

template <int MIX, int ADDR, int U, int SP, bool BUF>
static void run_flat(int T, int G, bool do_verify) {
  size_t slab = (N + G - 1) / G;
  const size_t q = (size_t)T * U;
  slab = (slab + q - 1) / q * q;
  if (do_verify && MIX != kRead) {
    for (int s = 0; s < 2; ++s) CK(hipMemset(buf[3 * s + 2], 0xee, N * 16));
  }
  const double us = median_us([&](int s) { flat<MIX, ADDR, U, SP, BUF><<<G, T>>>(buf[3 * s], buf[3 * s + 1], buf[3 * s + 2], N, slab); });
  const char* store = BUF ? "buffer-wt" : sp_name[SP];
  report(MIX, addr_name[ADDR], store, T, G, U, us, mix_bytes[MIX] * N * 16);
  if (do_verify) verify<MIX>((std::string(mix_name[MIX]) + " " + addr_name[ADDR] + " " + store).c_str(), N);
}

template <int MIX, int NW, int PPT, bool STAGED>
static void run_tiled(int G, bool do_verify) {
  constexpr size_t TP = 64 * NW * PPT;
  const size_t n_tiles = N / TP;   // the ragged rest of the tensor is left out
  if (do_verify) {
    for (int s = 0; s < 2; ++s) CK(hipMemset(buf[3 * s + 2], 0xee, N * 16));
  }
  const double us = median_us([&](int s) { tiled<MIX, NW, PPT, STAGED><<<G, 64 * NW>>>(buf[3 * s], buf[3 * s + 1], buf[3 * s + 2], n_tiles); });
  report(MIX, "tiles", STAGED ? "staged-1w" : "global-wt", 64 * NW, G, PPT, us, mix_bytes[MIX] * n_tiles * TP * 16);
  if (do_verify) verify<MIX>(STAGED ? "tiles staged" : "tiles own", n_tiles * TP);
}

template <int MIX, int ADDR, int SP, bool BUF>
static void sweep_flat(bool wide) {
  const int Ts[] = {256, 512, 1024};
  const int Gs_wide[] = {128, 192, 248, 256, 512}, Gs_narrow[] = {248, 256};
  bool first = true;
  for (int T : Ts)
    for (int gi = 0; gi < (wide ? 5 : 2); ++gi) {
      const int G = wide ? Gs_wide[gi] : Gs_narrow[gi];
      if (ADDR != kPairs) run_flat<MIX, ADDR, 1, SP, BUF>(T, G, first);
      run_flat<MIX, ADDR, 2, SP, BUF>(T, G, first && ADDR == kPairs);
      run_flat<MIX, ADDR, 4, SP, BUF>(T, G, false);
      first = false;
    }
}

template <int MIX>
static void sweep_mix() {
  sweep_flat<MIX, kStrided, 2, false>(true);
  if (MIX == kRead) return;
  sweep_flat<MIX, kChunk, 2, false>(false);
  sweep_flat<MIX, kSlab, 2, false>(false);
  sweep_flat<MIX, kPairs, 2, false>(false);
  sweep_flat<MIX, kStrided, 0, false>(false);
  sweep_flat<MIX, kStrided, 1, false>(false);
  sweep_flat<MIX, kStrided, 3, false>(false);
  sweep_flat<MIX, kStrided, 2, true>(false);
  if (MIX == kWrite) return;
  const int Gs[] = {248, 256};
  for (int G : Gs) {
    run_tiled<MIX, 10, 2, false>(G, G == 248);
    run_tiled<MIX, 10, 2, true>(G, G == 248);
    run_tiled<MIX, 8, 2, false>(G, false);
    run_tiled<MIX, 8, 2, true>(G, false);
    run_tiled<MIX, 5, 4, false>(G, false);
    run_tiled<MIX, 5, 4, true>(G, false);
    run_tiled<MIX, 16, 1, false>(G, false);
    run_tiled<MIX, 16, 1, true>(G, false);
  }
}

// Optional arguments: offsets in MiB by which the output buffers and the second input buffers are moved
// inside their (over-sized) allocations.  Bare streams with few loads in flight depend on where their
// buffers lie relative to one another (period 128 MiB), so a variant should be judged by its best placement.
int main(int argc, char** argv) {
  const size_t out_off = (argc > 1 ? strtoul(argv[1], nullptr, 10) : 0) << 20;
  const size_t in2_off = (argc > 2 ? strtoul(argv[2], nullptr, 10) : 0) << 20;
  const size_t slack = (size_t)160 << 20;
  for (int i = 0; i < 6; ++i) {
    const size_t off = i % 3 == 2 ? out_off : (i % 3 == 1 ? in2_off : 0);
    if (off > slack) { fprintf(stderr, "offset beyond %zu MiB\n", slack >> 20); return 2; }
    char* p = nullptr;
    CK(hipMalloc(&p, N * 16 + slack));
    buf[i] = reinterpret_cast<u32x4*>(p + off);
    CK(hipMemset(buf[i], 0x11 * (i + 1), N * 16));
  }
  printf("# output buffers moved by %zu MiB, second inputs by %zu MiB; (in - out) mod 128 MiB = %zu, %zu\n", out_off >> 20,
         in2_off >> 20, (size_t)(((uintptr_t)buf[0] - (uintptr_t)buf[2]) % ((size_t)128 << 20)) >> 20,
         (size_t)(((uintptr_t)buf[3] - (uintptr_t)buf[5]) % ((size_t)128 << 20)) >> 20);
  CK(hipMalloc(&bad, 8));
  // leave the idle power state before anything is timed
  for (int w = 0; w < 80; ++w) flat<kTwoReads, kStrided, 1, 2, false><<<256, 512>>>(buf[0], buf[1], buf[2], N, 0);
  CK(hipDeviceSynchronize());
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  printf("# %s, %d CUs, %zu bytes per stream\n", prop.name, prop.multiProcessorCount, N * 16);
  sweep_mix<kRead>();
  sweep_mix<kWrite>();
  sweep_mix<kCopy>();
  sweep_mix<kTwoReads>();
  printf("# best per (mix, address layout, store path)\n");
  for (const auto& kv : best) printf("best %s\n", kv.second.second.c_str());
  if (failures) {
    printf("# %d variant(s) produced wrong bytes\n", failures);
    return 1;
  }
  return 0;
}
