// C ABI of the fused normalisation kernels: argument validation, launch planning
// (variant, grid, workspace) and the kernel launches.  See include/teletron_op.h.
#include "teletron_op.h"

#include <atomic>
#include <initializer_list>
#include <mutex>
#include <unordered_map>

#include "generic_kernels.hpp"
#include "kernel_table.hpp"
#include "probe_kernels.hpp"

namespace tt {
namespace {

thread_local int g_last_hip_error = 0;

int hip_fail(hipError_t e) {
  g_last_hip_error = static_cast<int>(e);
  (void)hipGetLastError();  // clear the sticky launch error, it has been recorded
  return TT_ERR_HIP;
}

struct DeviceInfo {
  int cus = 0;
};

int current_device_cus(int* cus) {
  static std::mutex mu;
  static DeviceInfo info[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e);
  if (dev < 0 || dev >= 64) return TT_ERR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(mu);
  if (info[dev].cus == 0) {
    int n = 0;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return hip_fail(e);
    info[dev].cus = n > 0 ? n : 1;
  }
  *cus = info[dev].cus;
  return TT_OK;
}

// Resident workgroups per CU for a kernel, from the HIP occupancy calculator (cached).
int resident_wgs_per_cu(const KernelInfo& k, int* out) {
  static std::mutex mu;
  static std::unordered_map<const void*, int> cache;
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = cache.find(k.fn);
    if (it != cache.end()) { *out = it->second; return TT_OK; }
  }
  int n = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k.fn, k.threads, 0);
  if (e != hipSuccess) return hip_fail(e);
  if (n < 1) n = 1;
  std::lock_guard<std::mutex> lock(mu);
  cache[k.fn] = n;
  *out = n;
  return TT_OK;
}

// Backward workspace of tt_adaln_backward_static: a file-scope device array, so that the entry
// point never allocates.  Every device the library runs on holds its own copy at its own address;
// the host-side name below is only a handle for hipGetSymbolAddress, never a kernel argument.
static __device__ __align__(256) unsigned char scratch[TT_STATIC_WORKSPACE_BYTES];

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  static std::mutex mu;
  static void* addr[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e);
  if (dev < 0 || dev >= 64) return TT_ERR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e);
    if (!p) return TT_ERR_HIP;
    addr[dev] = p;
  }
  *out = addr[dev];
  return TT_OK;
}

std::atomic<int> g_wgs_per_cu_override{0};
std::atomic<int> g_grid_override{0};

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct Rope {
  const float* freqs = nullptr;
  int64_t head_dim = 0, seq_len = 0;
  int64_t heads = 0;   // 0: a row holds every head of a token; > 0: one head per row, `heads` rows per token
};

struct Plan {
  KernelInfo k;
  int64_t n_batches = 0;
  int64_t n_tiles = 0;   // per batch
  int grid_x = 0;        // workgroups per batch == partial sums per batch
  int packs = 0;
};

enum Dir { kFwd, kBwd, kBwdSaved, kFwdXn };   // kFwdXn: AdaLN forward that also stores x_norm
constexpr int kGateKind = 2;   // third op family next to kAdaLN / kRMS

// Upper bound on workgroups per batch used by any plan: what the workspace is sized for.
constexpr int kMaxWgsPerCu = 8;

// `res`: 0, or the residual + LayerNorm fusion: 1 plain, 2 gated (wide rows, kFwd / kBwd only).
int make_plan(int kind, Dir dir, int64_t rows, int64_t cols, int64_t rows_per_batch, Plan* plan, bool rope = false,
              int res = 0, int64_t rope_heads = 0) {
  if (rows <= 0 || cols <= 0 || rows_per_batch <= 0 || rows % rows_per_batch != 0)
    return TT_ERR_INVALID_ARGUMENT;
  if (cols > TT_MAX_COLS) return TT_ERR_UNSUPPORTED;
  if (cols % kPack != 0) return TT_ERR_UNSUPPORTED;
  const int packs = static_cast<int>(cols / kPack);
  const bool narrow = packs <= kNarrowMaxPacks;
  const int idx = narrow ? select_narrow(packs) : select_wide(packs);
  if (idx < 0) return TT_ERR_UNSUPPORTED;
  const int slots = narrow ? kNarrowL[idx] : 64 * kWideW[idx] * kWideP[idx];
  const bool full = (slots == packs);
  KernelInfo k;
  if (res) {
    if (narrow || kind != kAdaLN || dir == kBwdSaved || dir == kFwdXn) return TT_ERR_UNSUPPORTED;
    k = res == 2 ? resnorm_gated_kernel(dir == kBwd, idx, full) : resnorm_plain_kernel(dir == kBwd, idx, full);
  } else if (rope) {
    if (kind != kRMS || dir == kBwdSaved || dir == kFwdXn) return TT_ERR_UNSUPPORTED;
    k = rms_rope_kernel(narrow, dir == kBwd, idx, full, rope_heads);
  } else if (dir == kFwdXn) {
    if (kind != kAdaLN) return TT_ERR_UNSUPPORTED;
    k = adaln_fwd_xnorm_kernel(narrow, idx, full);
  } else if (kind == kAdaLN)
    k = dir == kFwd ? adaln_fwd_kernel(narrow, idx, full)
      : dir == kBwd ? adaln_bwd_kernel(narrow, idx, full) : adaln_bwd_saved_kernel(narrow, idx, full);
  else if (kind == kRMS)
    k = dir == kFwd ? rms_fwd_kernel(narrow, idx, full)
      : dir == kBwd ? rms_bwd_kernel(narrow, idx, full) : rms_bwd_saved_kernel(narrow, idx, full);
  else
    k = dir == kFwd ? gate_fwd_kernel(narrow, idx, full) : gate_bwd_kernel(narrow, idx, full);
  if (!k.fn) return TT_ERR_UNSUPPORTED;

  int cus = 0, per_cu = 0;
  int rc = current_device_cus(&cus);
  if (rc != TT_OK) return rc;
  rc = resident_wgs_per_cu(k, &per_cu);
  if (rc != TT_OK) return rc;
  // HBM streams fastest with a modest number of requests in flight: measured on MI355X,
  // throughput peaks near kFwdLoadsPerCu / kBwdLoadsPerCu outstanding 128-bit loads per lane
  // column of a CU (waves x loads per lane) and streamed tensor, falls off by 10-20 % at full
  // occupancy, and is a few percent better with one CU in 32 left without a workgroup.
  // Tensors that fit the caches just take the whole machine.
  const bool cache_resident = rows * cols * 2 < (int64_t)64 << 20;
  int usable_cus = cus;
  if (!cache_resident) {
    const int per_wg = (k.threads / kWave) * k.lane_loads;
    // two streamed inputs (backward kernels, both gate kernels) or one (normalisation forward)
    const int target = dir == kFwdXn ? kFwdXnLoadsPerCu
                     : (dir == kFwd && kind != kGateKind && !res) ? kFwdLoadsPerCu : kBwdLoadsPerCu;
    int want = (2 * target + per_wg) / (2 * per_wg);
    if (want < 1) want = 1;
    if (want < per_cu) per_cu = want;
    if (cus >= 32) usable_cus = cus - cus / 32;
  }
  const int ov = g_wgs_per_cu_override.load(std::memory_order_relaxed);
  if (ov > 0) per_cu = ov;
  if (per_cu > kMaxWgsPerCu) per_cu = kMaxWgsPerCu;

  plan->k = k;
  plan->packs = packs;
  plan->n_batches = rows / rows_per_batch;
  plan->n_tiles = (rows_per_batch + k.tile_rows - 1) / k.tile_rows;
  if (plan->n_batches > 65535) return TT_ERR_UNSUPPORTED;
  int64_t gx = (int64_t)per_cu * usable_cus / plan->n_batches;
  if (gx < 1) gx = 1;
  const int gov = g_grid_override.load(std::memory_order_relaxed);
  if (gov > 0 && gov <= kMaxWgsPerCu * cus) gx = gov / plan->n_batches > 0 ? gov / plan->n_batches : 1;
  if (gx > plan->n_tiles) gx = plan->n_tiles;
  plan->grid_x = static_cast<int>(gx);
  return TT_OK;
}

size_t partial_bytes(const Plan& p, int n_acc, int64_t cols) {
  return (size_t)p.n_batches * p.grid_x * n_acc * cols * sizeof(float);
}

// Workspace bound that does not depend on the launch-time occupancy query.
size_t workspace_bound(int n_acc, int64_t rows, int64_t cols, int64_t rows_per_batch) {
  if (rows <= 0 || cols <= 0 || rows_per_batch <= 0 || rows % rows_per_batch != 0) return 0;
  if (cols % kPack != 0) return (size_t)rows * 2 * sizeof(float);   // element-wise path: row statistics
  int cus = 0;
  if (current_device_cus(&cus) != TT_OK) cus = 256;
  const int64_t n_batches = rows / rows_per_batch;
  int64_t gx = (int64_t)kMaxWgsPerCu * cus / n_batches;
  if (gx < 1) gx = 1;
  if (gx > rows_per_batch) gx = rows_per_batch;
  return (size_t)n_batches * gx * n_acc * cols * sizeof(float);
}

// What the backward entry points of `kind` need for this shape: the partial sums of the plan they
// will actually launch (the larger of the two backward contracts).  Falls back to the
// plan-independent bound when a plan cannot be made here or a tuning override is active.
size_t workspace_for(int kind, int n_acc, int64_t rows, int64_t cols, int64_t rows_per_batch) {
  const size_t bound = workspace_bound(n_acc, rows, cols, rows_per_batch);
  if (bound == 0 || cols % kPack != 0) return bound;
  if (g_wgs_per_cu_override.load() > 0 || g_grid_override.load() > 0) return bound;
  Plan p;
  if (make_plan(kind, kBwd, rows, cols, rows_per_batch, &p) != TT_OK) return bound;
  size_t need = partial_bytes(p, n_acc, cols);
  if (kind != kGateKind && rows_per_batch == rows) {
    Plan ps;
    if (make_plan(kind, kBwdSaved, rows, cols, rows, &ps) != TT_OK) return bound;
    const size_t ns = partial_bytes(ps, n_acc, cols);
    if (ns > need) need = ns;
  }
  if (kind == kRMS) {   // tt_rmsnorm_rope[_heads]_backward share this size query: per-row and per-token kernels
    for (int64_t heads : {(int64_t)0, (int64_t)kRopeTokenHeads}) {
      Plan pr;
      if (make_plan(kRMS, kBwd, rows, cols, rows, &pr, true, 0, heads) == TT_OK) {
        const size_t nr = partial_bytes(pr, n_acc, cols);
        if (nr > need) need = nr;
      }
    }
  }
  return need < 16 ? 16 : need;
}

template <typename Args>
int launch(const Plan& p, Args& args, void* stream) {
  void* kargs[] = {&args};
  hipError_t e = hipLaunchKernel(p.k.fn, dim3(p.grid_x, (unsigned)p.n_batches, 1), dim3(p.k.threads, 1, 1),
                                 kargs, 0, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e);
  return TT_OK;
}

// ---------------------------------------------------------------- element-wise fallback
bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

int generic_grid(int64_t rows, int* grid) {
  int cus = 0;
  int rc = current_device_cus(&cus);
  if (rc != TT_OK) return rc;
  const int64_t cap = (int64_t)cus * 8;
  *grid = (int)(rows < cap ? rows : cap);
  return TT_OK;
}

int check_shape(int64_t rows, int64_t cols, int64_t rows_per_batch) {
  if (rows <= 0 || cols <= 0 || rows_per_batch <= 0 || rows % rows_per_batch != 0) return TT_ERR_INVALID_ARGUMENT;
  if (cols > TT_MAX_COLS || rows / rows_per_batch > 65535) return TT_ERR_UNSUPPORTED;
  return TT_OK;
}

int forward_generic(int kind, void* y, const void* x, const void* p0, const void* p1, float* mean, float* rstd,
                    void* x_norm, int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream) {
  int rc = check_shape(rows, cols, rows_per_batch);
  if (rc != TT_OK) return rc;
  if (!aligned2(y) || !aligned2(x) || !aligned2(p0) || !aligned2(p1) || !aligned2(x_norm)) return TT_ERR_INVALID_ARGUMENT;
  int grid = 0;
  rc = generic_grid(rows, &grid);
  if (rc != TT_OK) return rc;
  GenFwdArgs a;
  a.y = static_cast<uint16_t*>(y); a.x = static_cast<const uint16_t*>(x);
  a.p0 = static_cast<const uint16_t*>(p0); a.p1 = static_cast<const uint16_t*>(p1);
  a.mean = mean; a.rstd = rstd; a.x_norm = static_cast<uint16_t*>(x_norm);
  a.rows = rows; a.rows_per_batch = rows_per_batch; a.cols = (int)cols; a.eps = eps; a.inv_cols = 1.0f / (float)cols;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (kind == kAdaLN) hipLaunchKernelGGL(norm_fwd_generic<kAdaLN>, dim3(grid), dim3(kGenThreads), 0, s, a);
  else                hipLaunchKernelGGL(norm_fwd_generic<kRMS>, dim3(grid), dim3(kGenThreads), 0, s, a);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TT_OK : hip_fail(e);
}

int backward_generic(int kind, void* dx, void* out0, void* out1, const void* dy, const void* x, const void* p0,
                     void* workspace, size_t workspace_bytes, int64_t rows, int64_t cols, int64_t rows_per_batch,
                     float eps, void* stream) {
  int rc = check_shape(rows, cols, rows_per_batch);
  if (rc != TT_OK) return rc;
  if (!dx || !dy || !x || !p0 || !out0 || (kind == kAdaLN && !out1)) return TT_ERR_INVALID_ARGUMENT;
  if (!aligned2(dx) || !aligned2(dy) || !aligned2(x) || !aligned2(p0)) return TT_ERR_INVALID_ARGUMENT;
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 3u) != 0 ||
      workspace_bytes < (size_t)rows * 2 * sizeof(float))
    return TT_ERR_WORKSPACE;
  int grid = 0;
  rc = generic_grid(rows, &grid);
  if (rc != TT_OK) return rc;
  GenBwdArgs a;
  a.dx = static_cast<uint16_t*>(dx); a.dy = static_cast<const uint16_t*>(dy); a.x = static_cast<const uint16_t*>(x);
  a.p0 = static_cast<const uint16_t*>(p0); a.stats = static_cast<float*>(workspace); a.out0 = out0; a.out1 = out1;
  a.rows = rows; a.rows_per_batch = rows_per_batch; a.cols = (int)cols; a.eps = eps; a.inv_cols = 1.0f / (float)cols;
  a.out_bf16 = 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 cgrid((unsigned)((cols + 63) / 64), (unsigned)(rows / rows_per_batch), 1);
  if (kind == kAdaLN) {
    hipLaunchKernelGGL(norm_bwd_generic<kAdaLN>, dim3(grid), dim3(kGenThreads), 0, s, a);
    hipLaunchKernelGGL(norm_colgrad_generic<kAdaLN>, cgrid, dim3(1024), 0, s, a);
  } else {
    hipLaunchKernelGGL(norm_bwd_generic<kRMS>, dim3(grid), dim3(kGenThreads), 0, s, a);
    hipLaunchKernelGGL(norm_colgrad_generic<kRMS>, cgrid, dim3(1024), 0, s, a);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TT_OK : hip_fail(e);
}

// The vector kernels need 128-bit packs: cols % 8 == 0 and 16-byte aligned tensors.
bool vector_path(int64_t cols, std::initializer_list<const void*> ptrs) {
  if (cols % kPack != 0) return false;
  for (const void* p : ptrs)
    if (!aligned16(p)) return false;
  return true;
}

int check_rope(const Rope& rope, int64_t rows, int64_t cols) {
  if (!rope.freqs || rope.head_dim <= 0 || rope.seq_len <= 0 || rope.heads < 0) return TT_ERR_INVALID_ARGUMENT;
  if (rope.head_dim % kPack != 0 || rope.head_dim > 256 || cols % rope.head_dim != 0 || !aligned16(rope.freqs))
    return TT_ERR_UNSUPPORTED;
  if (rope.heads > 0) {   // one head per row: the narrow kernels
    if (cols != rope.head_dim) return TT_ERR_UNSUPPORTED;
    if (rows % rope.heads != 0) return TT_ERR_INVALID_ARGUMENT;
  } else if (cols / kPack <= kNarrowMaxPacks) {
    return TT_ERR_UNSUPPORTED;   // all heads in one row: the wide kernels
  }
  return TT_OK;
}

int forward(int kind, void* y, const void* x, const void* p0, const void* p1, float* mean, float* rstd, void* x_norm,
            int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream, const Rope* rope = nullptr) {
  if (rows == 0) return TT_OK;
  if (!y || !x || !p0 || (kind == kAdaLN && !p1)) return TT_ERR_INVALID_ARGUMENT;
  if (rope) {
    if (!vector_path(cols, {y, x, p0})) return TT_ERR_UNSUPPORTED;
    const int rrc = check_rope(*rope, rows, cols);
    if (rrc != TT_OK) return rrc;
  } else if (!vector_path(cols, {y, x, p0, p1, x_norm})) {
    return forward_generic(kind, y, x, p0, p1, mean, rstd, x_norm, rows, cols, rows_per_batch, eps, stream);
  }
  Plan p;
  if (x_norm && (kind != kAdaLN || rope)) return TT_ERR_UNSUPPORTED;
  int rc = make_plan(kind, x_norm ? kFwdXn : kFwd, rows, cols, rows_per_batch, &p, rope != nullptr, 0,
                     rope ? rope->heads : 0);
  if (rc != TT_OK) return rc;
  FwdArgs a;
  a.freqs = rope ? rope->freqs : nullptr; a.seq_len = rope ? rope->seq_len : 1; a.head_dim = rope ? (int)rope->head_dim : 8;
  a.rows_per_pos = rope && rope->heads > 0 ? rope->heads : 1;
  a.y = y; a.x = x; a.p0 = p0; a.p1 = p1; a.mean = mean; a.rstd = rstd; a.x_norm = x_norm;
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles;
  a.cols = (int)cols; a.packs = p.packs; a.eps = eps; a.inv_cols = 1.0f / (float)cols;
  return launch(p, a, stream);
}

int backward_partials(int kind, void* dx, const void* dy, const void* x, const void* p0,
                      void* workspace, size_t workspace_bytes, int* n_partials,
                      int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream,
                      const Rope* rope = nullptr) {
  if (n_partials) *n_partials = 0;
  if (rows == 0) return TT_OK;
  if (!dx || !dy || !x || !p0) return TT_ERR_INVALID_ARGUMENT;
  if (!aligned16(dx) || !aligned16(dy) || !aligned16(x) || !aligned16(p0)) return TT_ERR_UNSUPPORTED;
  if (rope) {
    const int rrc = check_rope(*rope, rows, cols);
    if (rrc != TT_OK) return rrc;
  }
  Plan p;
  int rc = make_plan(kind, kBwd, rows, cols, rows_per_batch, &p, rope != nullptr, 0, rope ? rope->heads : 0);
  if (rc != TT_OK) return rc;
  const int n_acc = kind == kAdaLN ? 2 : 1;
  if (!workspace || !aligned16(workspace) || workspace_bytes < partial_bytes(p, n_acc, cols)) return TT_ERR_WORKSPACE;
  BwdArgs a;
  a.freqs = rope ? rope->freqs : nullptr; a.seq_len = rope ? rope->seq_len : 1; a.head_dim = rope ? (int)rope->head_dim : 8;
  a.rows_per_pos = rope && rope->heads > 0 ? rope->heads : 1;
  a.dx = dx; a.dy = dy; a.x = x; a.p0 = p0; a.partials = static_cast<float*>(workspace);
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles;
  a.cols = (int)cols; a.packs = p.packs; a.eps = eps; a.inv_cols = 1.0f / (float)cols;
  rc = launch(p, a, stream);
  if (rc == TT_OK && n_partials) *n_partials = p.grid_x;
  return rc;
}

int backward_saved_partials(int kind, void* dx, const void* dy, const void* xs, const void* p0, const float* rstd,
                            void* workspace, size_t workspace_bytes, int* n_partials,
                            int64_t rows, int64_t cols, void* stream) {
  *n_partials = 0;
  if (rows == 0) return TT_OK;
  if (!dx || !dy || !xs || !p0 || !rstd) return TT_ERR_INVALID_ARGUMENT;
  if (!aligned16(dx) || !aligned16(dy) || !aligned16(xs) || !aligned16(p0)) return TT_ERR_UNSUPPORTED;
  Plan p;
  int rc = make_plan(kind, kBwdSaved, rows, cols, rows, &p);
  if (rc != TT_OK) return rc;
  const int n_acc = kind == kAdaLN ? 2 : 1;
  if (!workspace || !aligned16(workspace) || workspace_bytes < partial_bytes(p, n_acc, cols)) return TT_ERR_WORKSPACE;
  BwdSavedArgs a;
  a.dx = dx; a.dy = dy; a.xs = xs; a.p0 = p0; a.rstd = rstd; a.partials = static_cast<float*>(workspace);
  a.rows_per_batch = rows; a.n_tiles = p.n_tiles;
  a.cols = (int)cols; a.packs = p.packs; a.inv_cols = 1.0f / (float)cols;
  rc = launch(p, a, stream);
  if (rc == TT_OK) *n_partials = p.grid_x;
  return rc;
}

int reduce(void* out0, void* out1, const void* workspace, int n_batches, int n_partials, int n_acc,
           int64_t cols, bool out_bf16, void* stream, void* out2 = nullptr) {
  if (n_batches == 0) return TT_OK;
  if (!out0 || !workspace || n_batches < 0 || n_batches > 65535 || n_partials <= 0 || cols <= 0 ||
      cols > TT_MAX_COLS || n_acc < 1 || n_acc > 3 || (n_acc >= 2 && !out1) || (n_acc == 3 && !out2))
    return TT_ERR_INVALID_ARGUMENT;
  const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)n_batches, 1);
  const float* ws = static_cast<const float*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int bf = out_bf16 ? 1 : 0;
  if (n_acc == 3)      hipLaunchKernelGGL(reduce_partials<3>, grid, dim3(1024), 0, s, out0, out1, out2, ws, n_partials, (int)cols, bf);
  else if (n_acc == 2) hipLaunchKernelGGL(reduce_partials<2>, grid, dim3(1024), 0, s, out0, out1, out2, ws, n_partials, (int)cols, bf);
  else                 hipLaunchKernelGGL(reduce_partials<1>, grid, dim3(1024), 0, s, out0, out1, out2, ws, n_partials, (int)cols, bf);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return TT_OK;
}

}  // namespace
}  // namespace tt

using namespace tt;

extern "C" {

int tt_version(void) { return 100; }

const char* tt_error_string(int code) {
  switch (code) {
    case TT_OK: return "ok";
    case TT_ERR_INVALID_ARGUMENT: return "invalid argument (null pointer, non-positive size, or rows not a multiple of rows_per_batch)";
    case TT_ERR_UNSUPPORTED: return "unsupported shape or alignment";
    case TT_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case TT_ERR_HIP: return "HIP runtime error (see tt_last_hip_error)";
    case TT_ERR_STATIC_LIMIT: return "shape needs more than TT_STATIC_WORKSPACE_BYTES of scratch (partial sums, or rows * 8 bytes on the element-wise path): use the entry point that takes a workspace";
    default: return "unknown error code";
  }
}

int tt_last_hip_error(void) { return g_last_hip_error; }

#ifdef TT_TUNING_HOOKS
// Tuning hooks, compiled only into sweep builds (not part of the public header): force the number
// of resident workgroups per CU that launch plans assume, or the total number of workgroups of a
// launch; 0 restores the plan's own choice.
TT_API void tt_debug_set_wgs_per_cu(int n) { g_wgs_per_cu_override.store(n < 0 ? 0 : n); }
TT_API void tt_debug_set_grid(int n) { g_grid_override.store(n < 0 ? 0 : n); }
#endif

int tt_adaln_forward(void* y, const void* x, const void* scale, const void* shift, float* mean, float* rstd,
                     int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream) {
  return forward(kAdaLN, y, x, scale, shift, mean, rstd, nullptr, rows, cols, rows_per_batch, eps, stream);
}

int tt_rmsnorm_forward(void* y, const void* x, const void* weight, float* rstd,
                       int64_t rows, int64_t cols, float eps, void* stream) {
  return forward(kRMS, y, x, weight, nullptr, nullptr, rstd, nullptr, rows, cols, rows, eps, stream);
}

size_t tt_adaln_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch) {
  return workspace_for(kAdaLN, 2, rows, cols, rows_per_batch);
}
size_t tt_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols) {
  return workspace_for(kRMS, 1, rows, cols, rows);
}

int tt_adaln_backward_partials(void* dx, const void* dy, const void* x, const void* scale,
                               void* workspace, size_t workspace_bytes, int* n_partials,
                               int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream) {
  return backward_partials(kAdaLN, dx, dy, x, scale, workspace, workspace_bytes, n_partials,
                           rows, cols, rows_per_batch, eps, stream);
}
int tt_rmsnorm_backward_partials(void* dx, const void* dy, const void* x, const void* weight,
                                 void* workspace, size_t workspace_bytes, int* n_partials,
                                 int64_t rows, int64_t cols, float eps, void* stream) {
  return backward_partials(kRMS, dx, dy, x, weight, workspace, workspace_bytes, n_partials,
                           rows, cols, rows, eps, stream);
}

int tt_reduce_partials(float* out0, float* out1, const void* workspace,
                       int n_batches, int n_partials, int n_acc, int64_t cols, void* stream) {
  return reduce(out0, out1, workspace, n_batches, n_partials, n_acc, cols, false, stream);
}

int tt_adaln_backward(void* dx, float* dscale, float* dshift, const void* dy, const void* x, const void* scale,
                      void* workspace, size_t workspace_bytes,
                      int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dscale || !dshift) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {dx, dy, x, scale, workspace}))
    return backward_generic(kAdaLN, dx, dscale, dshift, dy, x, scale, workspace, workspace_bytes,
                            rows, cols, rows_per_batch, eps, stream);
  int n_partials = 0;
  int rc = backward_partials(kAdaLN, dx, dy, x, scale, workspace, workspace_bytes, &n_partials,
                             rows, cols, rows_per_batch, eps, stream);
  if (rc != TT_OK) return rc;
  return reduce(dscale, dshift, workspace, (int)(rows / rows_per_batch), n_partials, 2, cols, false, stream);
}

int tt_adaln_backward_static(void* dx, float* dscale, float* dshift, const void* dy, const void* x,
                             const void* scale, int64_t rows, int64_t cols, int64_t rows_per_batch, float eps,
                             void* stream) {
  void* ws = nullptr;
  int rc = static_scratch(&ws);   // per-device set-up on the first call; a rows == 0 call does only this
  if (rc != TT_OK) return rc;
  if (rows == 0) return TT_OK;
  rc = tt_adaln_backward(dx, dscale, dshift, dy, x, scale, ws, TT_STATIC_WORKSPACE_BYTES,
                         rows, cols, rows_per_batch, eps, stream);
  return rc == TT_ERR_WORKSPACE ? TT_ERR_STATIC_LIMIT : rc;
}

int tt_rmsnorm_backward(void* dx, float* dweight, const void* dy, const void* x, const void* weight,
                        void* workspace, size_t workspace_bytes,
                        int64_t rows, int64_t cols, float eps, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dweight) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {dx, dy, x, weight, workspace}))
    return backward_generic(kRMS, dx, dweight, nullptr, dy, x, weight, workspace, workspace_bytes,
                            rows, cols, rows, eps, stream);
  int n_partials = 0;
  int rc = backward_partials(kRMS, dx, dy, x, weight, workspace, workspace_bytes, &n_partials,
                             rows, cols, rows, eps, stream);
  if (rc != TT_OK) return rc;
  return reduce(dweight, nullptr, workspace, 1, n_partials, 1, cols, false, stream);
}

// ---------------------------------------------------------------- RMSNorm + rotary embedding
int tt_rmsnorm_rope_forward(void* y, const void* x, const void* weight, const float* freqs, float* rstd,
                            int64_t rows, int64_t cols, int64_t head_dim, int64_t seq_len, float eps, void* stream) {
  Rope rope; rope.freqs = freqs; rope.head_dim = head_dim; rope.seq_len = seq_len;
  return forward(kRMS, y, x, weight, nullptr, nullptr, rstd, nullptr, rows, cols, rows, eps, stream, &rope);
}

int tt_rmsnorm_rope_backward(void* dx, float* dweight, const void* dy, const void* x, const void* weight,
                             const float* freqs, void* workspace, size_t workspace_bytes,
                             int64_t rows, int64_t cols, int64_t head_dim, int64_t seq_len, float eps, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dweight) return TT_ERR_INVALID_ARGUMENT;
  Rope rope; rope.freqs = freqs; rope.head_dim = head_dim; rope.seq_len = seq_len;
  int n_partials = 0;
  int rc = backward_partials(kRMS, dx, dy, x, weight, workspace, workspace_bytes, &n_partials,
                             rows, cols, rows, eps, stream, &rope);
  if (rc != TT_OK) return rc;
  return reduce(dweight, nullptr, workspace, 1, n_partials, 1, cols, false, stream);
}

int tt_rmsnorm_rope_heads_forward(void* y, const void* x, const void* weight, const float* freqs, float* rstd,
                                  int64_t rows, int64_t head_dim, int64_t heads, int64_t seq_len, float eps,
                                  void* stream) {
  if (heads <= 0) return TT_ERR_INVALID_ARGUMENT;
  Rope rope; rope.freqs = freqs; rope.head_dim = head_dim; rope.seq_len = seq_len; rope.heads = heads;
  return forward(kRMS, y, x, weight, nullptr, nullptr, rstd, nullptr, rows, head_dim, rows, eps, stream, &rope);
}

int tt_rmsnorm_rope_heads_backward(void* dx, float* dweight, const void* dy, const void* x, const void* weight,
                                   const float* freqs, void* workspace, size_t workspace_bytes,
                                   int64_t rows, int64_t head_dim, int64_t heads, int64_t seq_len, float eps,
                                   void* stream) {
  if (rows == 0) return TT_OK;
  if (!dweight || heads <= 0) return TT_ERR_INVALID_ARGUMENT;
  Rope rope; rope.freqs = freqs; rope.head_dim = head_dim; rope.seq_len = seq_len; rope.heads = heads;
  int n_partials = 0;
  int rc = backward_partials(kRMS, dx, dy, x, weight, workspace, workspace_bytes, &n_partials,
                             rows, head_dim, rows, eps, stream, &rope);
  if (rc != TT_OK) return rc;
  return reduce(dweight, nullptr, workspace, 1, n_partials, 1, head_dim, false, stream);
}

// ---------------------------------------------------------------- gated residual add
int tt_gate_residual_forward(void* out, const void* x, const void* gate, const void* residual,
                             int64_t rows, int64_t cols, int64_t rows_per_batch, void* stream) {
  if (rows == 0) return TT_OK;
  if (!out || !x || !gate || !residual) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {out, x, gate, residual})) return TT_ERR_UNSUPPORTED;
  Plan p;
  int rc = make_plan(kGateKind, kFwd, rows, cols, rows_per_batch, &p);
  if (rc != TT_OK) return rc;
  GateArgs a;
  a.out = out; a.a = x; a.b = residual; a.gate = gate; a.partials = nullptr;
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles; a.cols = (int)cols; a.packs = p.packs;
  return launch(p, a, stream);
}

size_t tt_gate_residual_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch) {
  return cols % kPack == 0 ? workspace_for(kGateKind, 1, rows, cols, rows_per_batch) : 0;
}

int tt_gate_residual_backward(void* dresidual, float* dgate, const void* dout, const void* gate,
                              const void* residual, void* workspace, size_t workspace_bytes,
                              int64_t rows, int64_t cols, int64_t rows_per_batch, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dresidual || !dgate || !dout || !gate || !residual) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {dresidual, dout, gate, residual})) return TT_ERR_UNSUPPORTED;
  Plan p;
  int rc = make_plan(kGateKind, kBwd, rows, cols, rows_per_batch, &p);
  if (rc != TT_OK) return rc;
  if (!workspace || !aligned16(workspace) || workspace_bytes < partial_bytes(p, 1, cols)) return TT_ERR_WORKSPACE;
  GateArgs a;
  a.out = dresidual; a.a = dout; a.b = residual; a.gate = gate; a.partials = static_cast<float*>(workspace);
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles; a.cols = (int)cols; a.packs = p.packs;
  rc = launch(p, a, stream);
  if (rc != TT_OK) return rc;
  return reduce(dgate, nullptr, workspace, (int)(rows / rows_per_batch), p.grid_x, 1, cols, false, stream);
}

// ---------------------------------------------------------------- residual update + LayerNorm
// scale / shift / gate hold either one vector for all batches or one per batch.
static bool stride_ok(int64_t n_vectors, int64_t n_batches) { return n_vectors == 1 || n_vectors == n_batches; }

int tt_residual_norm_forward(void* s, void* y, const void* x, const void* r, const void* gate, int64_t n_gate,
                             const void* scale, const void* shift, int64_t n_param, int affine,
                             float* mean, float* rstd, int64_t rows, int64_t cols, int64_t rows_per_batch,
                             float eps, void* stream) {
  if (rows == 0) return TT_OK;
  if (!s || !y || !x || !r || !scale || !shift) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {s, y, x, r, gate, scale, shift})) return TT_ERR_UNSUPPORTED;
  Plan p;
  int rc = make_plan(kAdaLN, kFwd, rows, cols, rows_per_batch, &p, false, gate ? 2 : 1);
  if (rc != TT_OK) return rc;
  if (!stride_ok(n_param, p.n_batches) || (gate && !stride_ok(n_gate, p.n_batches))) return TT_ERR_INVALID_ARGUMENT;
  ResFwdArgs a;
  a.s = s; a.y = y; a.x = x; a.r = r; a.gate = gate; a.scale = scale; a.shift = shift; a.mean = mean; a.rstd = rstd;
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles;
  a.gate_stride = n_gate == 1 ? 0 : cols; a.param_stride = n_param == 1 ? 0 : cols;
  a.cols = (int)cols; a.packs = p.packs; a.eps = eps; a.inv_cols = 1.0f / (float)cols; a.one = affine ? 0.f : 1.f;
  return launch(p, a, stream);
}

size_t tt_residual_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch, int gated) {
  if (rows <= 0 || cols <= 0 || cols % kPack != 0) return 0;
  Plan p;
  if (make_plan(kAdaLN, kBwd, rows, cols, rows_per_batch, &p, false, gated ? 2 : 1) != TT_OK) return 0;
  if (g_wgs_per_cu_override.load() > 0 || g_grid_override.load() > 0)
    return workspace_bound(gated ? 3 : 2, rows, cols, rows_per_batch);
  const size_t need = partial_bytes(p, gated ? 3 : 2, cols);
  return need < 16 ? 16 : need;
}

int tt_residual_norm_backward(void* dx, void* dr, float* dscale, float* dshift, float* dgate,
                              const void* dy, const void* ds_in, const void* s, const void* r,
                              const void* gate, int64_t n_gate, const void* scale, int64_t n_param, int affine,
                              void* workspace, size_t workspace_bytes,
                              int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream) {
  if (rows == 0) return TT_OK;
  const bool gated = gate != nullptr;
  if (!dx || !dscale || !dshift || !dy || !s || !scale) return TT_ERR_INVALID_ARGUMENT;
  if (gated && (!dr || !dgate || !r)) return TT_ERR_INVALID_ARGUMENT;
  if (!vector_path(cols, {dx, dr, dy, ds_in, s, r, gate, scale})) return TT_ERR_UNSUPPORTED;
  Plan p;
  int rc = make_plan(kAdaLN, kBwd, rows, cols, rows_per_batch, &p, false, gated ? 2 : 1);
  if (rc != TT_OK) return rc;
  if (!stride_ok(n_param, p.n_batches) || (gated && !stride_ok(n_gate, p.n_batches))) return TT_ERR_INVALID_ARGUMENT;
  const int n_acc = gated ? 3 : 2;
  if (!workspace || !aligned16(workspace) || workspace_bytes < partial_bytes(p, n_acc, cols)) return TT_ERR_WORKSPACE;
  ResBwdArgs a;
  a.dx = dx; a.dr = dr; a.dy = dy; a.ds_in = ds_in; a.s = s; a.r = r; a.gate = gate; a.scale = scale;
  a.partials = static_cast<float*>(workspace);
  a.rows_per_batch = rows_per_batch; a.n_tiles = p.n_tiles;
  a.gate_stride = n_gate == 1 ? 0 : cols; a.param_stride = n_param == 1 ? 0 : cols;
  a.cols = (int)cols; a.packs = p.packs; a.eps = eps; a.inv_cols = 1.0f / (float)cols; a.one = affine ? 0.f : 1.f;
  rc = launch(p, a, stream);
  if (rc != TT_OK) return rc;
  return reduce(dscale, dshift, workspace, (int)p.n_batches, p.grid_x, n_acc, cols, false, stream, dgate);
}

// ---------------------------------------------------------------- bare streaming probe
int tt_stream_probe(void* out, const void* a, const void* b, size_t bytes, void* stream) {
  if (bytes == 0) return TT_OK;
  if ((!out && !a) || (b && (!out || !a))) return TT_ERR_INVALID_ARGUMENT;
  if (bytes % 16 != 0 || !aligned16(out) || !aligned16(a) || !aligned16(b)) return TT_ERR_UNSUPPORTED;
  int cus = 0;
  const int rc = current_device_cus(&cus);
  if (rc != TT_OK) return rc;
  const size_t n = bytes / 16;
  // One workgroup per CU; threads and packs per lane in flight are what streamed fastest for each
  // mix on MI355X (reads want many requests in flight, writes few: 4 waves with one store each).
  const int threads = !a ? 256 : kProbeMaxThreads;
  const size_t want = (n + threads - 1) / threads;
  // two reads per write stream best with one CU in 32 left without a workgroup, like the kernels
  const size_t wgs = (b && cus >= 32) ? (size_t)(cus - cus / 32) : (size_t)cus;
  const dim3 grid((unsigned)(want < wgs ? want : wgs));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!out)    hipLaunchKernelGGL((stream_probe<kProbeRead, 4>), grid, dim3(threads), 0, s, out, a, b, n);
  else if (!a) hipLaunchKernelGGL((stream_probe<kProbeWrite, 1>), grid, dim3(threads), 0, s, out, a, b, n);
  else if (b)  hipLaunchKernelGGL((stream_probe<kProbeXor, 1>), grid, dim3(threads), 0, s, out, a, b, n);
  else         hipLaunchKernelGGL((stream_probe<kProbeCopy, 2>), grid, dim3(threads), 0, s, out, a, b, n);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? TT_OK : hip_fail(e);
}

int tt_stream_probe_two_outputs(void* out0, void* out1, const void* a, size_t bytes, void* stream) {
  if (bytes == 0) return TT_OK;
  if (!out0 || !out1 || !a) return TT_ERR_INVALID_ARGUMENT;
  if (bytes % 16 != 0 || !aligned16(out0) || !aligned16(out1) || !aligned16(a)) return TT_ERR_UNSUPPORTED;
  int cus = 0;
  const int rc = current_device_cus(&cus);
  if (rc != TT_OK) return rc;
  // four waves per CU with four packs per lane in flight streamed this mix fastest on MI355X
  constexpr int kThreads = 256, kU = 4;
  const size_t n = bytes / 16;
  const size_t tiles = (n + kThreads * kU - 1) / (kThreads * kU);
  const dim3 grid((unsigned)(tiles < (size_t)cus ? tiles : (size_t)cus));
  hipLaunchKernelGGL((stream_probe_two_outputs<kU>), grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     out0, out1, a, n);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? TT_OK : hip_fail(e);
}

// ---------------------------------------------------------------- reference-compatible contract
int tt_launch_adaln_forward(void* output, void* x_norm, const void* input, const void* scale, const void* shift,
                            int64_t rows, int64_t cols, double epsilon, float* inv_variance, void* stream) {
  if (rows != 0 && (!x_norm || !inv_variance)) return TT_ERR_INVALID_ARGUMENT;
  return forward(kAdaLN, output, input, scale, shift, nullptr, inv_variance, x_norm, rows, cols, rows,
                 static_cast<float>(epsilon), stream);
}

int tt_launch_adaln_backward(void* dinp, void* dscale, void* dshift, const void* dout, const void* x_norm,
                             const void* scale, const float* inv_variance, int64_t rows, int64_t cols,
                             void* workspace, size_t workspace_bytes, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dscale || !dshift) return TT_ERR_INVALID_ARGUMENT;
  int n_partials = 0;
  int rc = backward_saved_partials(kAdaLN, dinp, dout, x_norm, scale, inv_variance, workspace, workspace_bytes,
                                   &n_partials, rows, cols, stream);
  if (rc != TT_OK) return rc;
  return reduce(dscale, dshift, workspace, 1, n_partials, 2, cols, true, stream);
}

int tt_launch_rms_forward(void* output, const void* input, const void* weight, int64_t rows, int64_t cols,
                          double epsilon, float* inv_variance, void* stream) {
  if (rows != 0 && !inv_variance) return TT_ERR_INVALID_ARGUMENT;
  return forward(kRMS, output, input, weight, nullptr, nullptr, inv_variance, nullptr, rows, cols, rows,
                 static_cast<float>(epsilon), stream);
}

int tt_launch_rms_backward(void* dinp, void* dweight, const void* dout, const void* x_rmsnorm, const void* weight,
                           const float* inv_variance, int64_t rows, int64_t cols,
                           void* workspace, size_t workspace_bytes, void* stream) {
  if (rows == 0) return TT_OK;
  if (!dweight) return TT_ERR_INVALID_ARGUMENT;
  int n_partials = 0;
  int rc = backward_saved_partials(kRMS, dinp, dout, x_rmsnorm, weight, inv_variance, workspace, workspace_bytes,
                                   &n_partials, rows, cols, stream);
  if (rc != TT_OK) return rc;
  return reduce(dweight, nullptr, workspace, 1, n_partials, 1, cols, true, stream);
}

}  // extern "C"
