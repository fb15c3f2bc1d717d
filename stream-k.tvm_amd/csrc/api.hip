// C ABI of libstreamk.so: argument checking, workspace carving, kernel launch.
#include <hip/hip_runtime.h>

#include <mutex>
#include <unordered_map>

#include "launch.h"
#include "q4_dequant.h"
#include "streamk.h"

using namespace sk;

namespace {

struct DeviceInfo {
  int ok = 0, cus = 0, clock_khz = 0, lds = 0;
};
// one mutex guards every lazily filled table of this file (device properties, occupancies, the
// workspace registry): the entry points may be called from several host threads
std::mutex g_mutex;

DeviceInfo device_info() {
  static DeviceInfo d[16];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return DeviceInfo();
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!d[dev].ok) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, dev) == hipSuccess) {
      d[dev].cus = p.multiProcessorCount;
      d[dev].clock_khz = p.clockRate;
      d[dev].lds = (int)p.maxSharedMemoryPerMultiProcessor;
      d[dev].ok = 1;
    }
  }
  return d[dev];
}

__global__ void fill_zero_kernel(uint32_t *p, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = 0;
}

// Whether the partial area holds leftovers is recorded in the workspace itself, not on the host, so
// that a launch replayed from a graph sees what actually ran before it.  Kernels leave flags and
// counters at zero.  ATOMIC launches need the accumulators they add into zeroed and leave them
// zeroed; REDUCE launches leave partial tiles behind and raise the high-water mark status[WS_DIRTY]
// (in 256-byte units from the start of the partial area) past every slot they write.  This kernel
// runs in front of every ATOMIC launch: with the mark at zero it returns at once; otherwise it
// zero-fills the area up to the mark (as far as the caller's buffer reaches) and the block that
// finishes last lowers the mark again.
__global__ void clean_partials_kernel(int *status, uint4v *partials, unsigned capacity_units) {
  const unsigned mark = (unsigned)__hip_atomic_load(status + WS_DIRTY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (mark == 0) return;
  const size_t n16 = (size_t)(mark < capacity_units ? mark : capacity_units) * 16;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) partials[i] = uint4v{0, 0, 0, 0};
  __syncthreads();  // every thread of the block has read the mark
  if (threadIdx.x == 0) {
    const int done = __hip_atomic_fetch_add(status + WS_CLEAN_DONE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (done == (int)gridDim.x - 1) {
      __hip_atomic_store(status + WS_CLEAN_DONE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // a mark beyond this caller's buffer stays: a later call with the larger buffer cleans the rest
      if (mark <= capacity_units) __hip_atomic_store(status + WS_DIRTY, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Workspaces the library has initialised (sk_workspace_init) and not been told to forget
// (sk_workspace_release).  `poisoned` is set when sk_workspace_status has seen a timed-out fix-up
// wait: flags of that launch may still be raised, so further launches are refused until the
// workspace is initialised again.
struct WsInfo {
  size_t bytes;
  bool poisoned;
  // host-side hint: a launch enqueued through this library may have left partial tiles in the workspace (the
  // authoritative record is the dirty mark in the workspace itself; a stale hint only costs time)
  bool maybe_dirty;
};
std::unordered_map<const void *, WsInfo> g_ws;

// Workspace of sk_gemm_f16_static, for callers that must not allocate: one array per device, part of
// the code object (zero-filled when the module is loaded), laid out like a caller's workspace.  In host
// code its name is only a handle: the address kernels are given comes from hipGetSymbolAddress, once
// per device, and is kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[SK_STATIC_WORKSPACE_BYTES];
void *g_scratch_ptr[16];

int static_scratch(void **ptr) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return SK_ERR_DEVICE;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return SK_ERR_DEVICE;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return SK_OK;
}

// Runs in front of every launch on the static workspace, whose contents are whatever the previous call
// left: clears the status word and the flags / counters the plan uses (an abandoned wait of an earlier
// call may have left some raised) and, for an ATOMIC plan, zero-fills the partial area as far as it is
// marked dirty (see clean_partials_kernel).
__global__ void prepare_static_kernel(int *status, int *flags, int nflags, uint4v *partials, unsigned capacity_units,
                                      int atomic) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
  if (tid == 0) status[WS_STATUS] = 0;
  for (size_t i = tid; i < (size_t)nflags; i += stride) flags[i] = 0;
  if (!atomic) return;
  const unsigned mark = (unsigned)__hip_atomic_load(status + WS_DIRTY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (mark == 0) return;
  const size_t n16 = (size_t)(mark < capacity_units ? mark : capacity_units) * 16;
  for (size_t i = tid; i < n16; i += stride) partials[i] = uint4v{0, 0, 0, 0};
  __syncthreads();
  if (threadIdx.x == 0) {
    const int done = __hip_atomic_fetch_add(status + WS_CLEAN_DONE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (done == (int)gridDim.x - 1) {
      __hip_atomic_store(status + WS_CLEAN_DONE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (mark <= capacity_units) __hip_atomic_store(status + WS_DIRTY, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// zero-fill of a 16-bit C, two elements per store (rows of `pairs` pairs, `ld` pairs apart), for the fix-up that adds
// its partial tiles into C
__global__ void zero_pairs_kernel(uint32_t *C, int M, int pairs, int64_t ld) {
  const int64_t total = (int64_t)M * pairs;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / pairs;
    C[r * ld + (i - r * pairs)] = 0u;
  }
}

// the ordered reduce, with fp32 or 16-bit partial tiles
static inline bool is_reduce(int fixup) { return fixup == SK_FIXUP_REDUCE || fixup == SK_FIXUP_REDUCE16; }

int check_plan(const sk_plan *plan, int64_t M, int64_t N, int64_t K, int dtype, int layout) {
  if (!plan) return SK_ERR_NULL;
  if (plan->M != M || plan->N != N || plan->K != K || plan->dtype != dtype || plan->layout != layout)
    return SK_ERR_CONFIG;
  return SK_OK;
}

// is_static: ws is the library's own static workspace (no registry entry; prepared by its own kernel)
int make_dev_plan(const sk_plan *plan, const KernelInfo *k, void *ws, size_t ws_bytes, int occupancy,
                  hipStream_t stream, DevPlan *dp, Workspace *w, bool is_static = false) {
  if ((size_t)plan->workspace_bytes > ws_bytes) return SK_ERR_WORKSPACE;
  if (plan->workspace_bytes > 0 && !ws) return SK_ERR_WORKSPACE;
  if (plan->workspace_bytes > 0 && (reinterpret_cast<uintptr_t>(ws) & 255)) return SK_ERR_ALIGN;
  const DeviceInfo d = device_info();
  if (!d.ok) return SK_ERR_DEVICE;
  // every CTA of the Stream-K wave may wait on another one: they must all be resident
  if (plan->streamk_tiles > 0 && is_reduce(plan->fixup) &&
      (occupancy <= 0 || plan->grid > d.cus * occupancy))
    return SK_ERR_CONFIG;
  if (plan->workspace_bytes > 0 && is_static) {
    char *base = static_cast<char *>(ws);
    // (REDUCE: one flag per CTA, and a second one for the two-round exchange of tiles cut into four)
    const int nflags = is_reduce(plan->fixup) ? 2 * plan->grid : plan->streamk_tiles;
    const size_t units = (ws_bytes - (size_t)WS_PART_OFF) / 256;
    hipLaunchKernelGGL(prepare_static_kernel, dim3(1024), dim3(256), 0, stream, reinterpret_cast<int *>(base),
                       reinterpret_cast<int *>(base + 256), nflags, reinterpret_cast<uint4v *>(base + WS_PART_OFF),
                       (unsigned)units, plan->fixup == SK_FIXUP_ATOMIC ? 1 : 0);
    if (hipGetLastError() != hipSuccess) return SK_ERR_LAUNCH;
  } else if (plan->workspace_bytes > 0) {
    bool wide_clean = false;
    size_t registered_bytes = ws_bytes;
    {
      std::lock_guard<std::mutex> lock(g_mutex);
      auto it = g_ws.find(ws);
      if (it == g_ws.end() || it->second.bytes < ws_bytes) return SK_ERR_WORKSPACE;  // sk_workspace_init was never run on it
      if (it->second.poisoned) return SK_ERR_TIMEOUT;
      registered_bytes = it->second.bytes;
      if (plan->fixup == SK_FIXUP_ATOMIC) {
        wide_clean = it->second.maybe_dirty;
        it->second.maybe_dirty = false;
      } else if (is_reduce(plan->fixup) && plan->streamk_tiles > 0) {
        it->second.maybe_dirty = true;
      }
    }
    if (plan->fixup == SK_FIXUP_ATOMIC) {
      // The cleaner reads the mark the workspace carries and returns at once when it is zero.  Where this library has
      // not enqueued anything that could have raised it, one small block does that; it still cleans correctly (only
      // slowly) if a captured REDUCE launch replayed in between proves the hint wrong.
      // (the capacity is that of the workspace as it was initialised, not of this call's share of it: the mark can
      // then never lie beyond what the cleaner may touch, and a cleaned workspace always reads as clean)
      char *base = static_cast<char *>(ws);
      const size_t units = (registered_bytes - (size_t)WS_PART_OFF) / 256;
      hipLaunchKernelGGL(clean_partials_kernel, dim3(wide_clean ? 1024 : 1), dim3(256), 0, stream, reinterpret_cast<int *>(base),
                         reinterpret_cast<uint4v *>(base + WS_PART_OFF), (unsigned)(units > 0xffffffffu ? 0xffffffffu : units));
      if (hipGetLastError() != hipSuccess) return SK_ERR_LAUNCH;
    }
  }
  dp->tiles_m = plan->num_block_m;
  dp->tiles_n = plan->num_block_n;
  dp->ipt = plan->iters_per_tile;
  dp->total_tiles = plan->total_tiles;
  dp->sk_tiles = plan->streamk_tiles;
  dp->sk_full = plan->streamk_full_tiles;
  dp->sk_extra = plan->streamk_partial_tiles;
  dp->grid = plan->grid;
  dp->fixup = plan->fixup == SK_FIXUP_ATOMIC ? FIXUP_ATOMIC : (plan->fixup == SK_FIXUP_ATOMIC_C ? FIXUP_ATOMIC_C : FIXUP_REDUCE);
  dp->raster = plan->raster;
  dp->spin_limit = plan->spin_limit > 0 ? plan->spin_limit : (1 << 22);
  // (the interleaved Stream-K order relies on the hardware's round-robin placement: CTAs a multiple of 8 apart
  // share an XCD)
  dp->xcd_remap = plan->interleave <= 1 ? 1 : 0;
  dp->perm_s = plan->interleave > 1 ? plan->interleave : 1;
  dp->perm_g = plan->interleave > 1 ? plan->streamk_tiles / plan->interleave : 1;
  dp->by_perm = FastDiv::make(dp->perm_s);
  const int raster = plan->raster > 0 ? plan->raster : 1;
  dp->raster_tail = plan->num_block_m % raster ? plan->num_block_m % raster : raster;
  // every Stream-K tile cut into exactly two equal CTA segments: both CTAs of a pair finish half a tile
  dp->halves = 0;
  if (is_reduce(plan->fixup) && plan->streamk_tiles > 0 && plan->streamk_partial_tiles == 0) {
    if (2 * plan->streamk_full_tiles == plan->iters_per_tile) dp->halves = 1;
    // four equal segments: two rounds of the same exchange (the second round's flags follow the first `grid` ones)
    if (4 * plan->streamk_full_tiles == plan->iters_per_tile && 2 * (int64_t)plan->grid <= WS_MAX_FLAGS) dp->halves = 2;
  }
  dp->partials16 = 0;
  if (plan->fixup == SK_FIXUP_REDUCE16) {
    // (a plan that sk_make_plan would not have made: refuse it rather than run another fix-up than it names)
    if (!(dp->halves > 0 && k->family == FAMILY_TILE && k->variant == 7 && (plan->dtype == SK_F16 || plan->dtype == SK_BF16)))
      return SK_ERR_CONFIG;
    dp->partials16 = 1;
  }
  dp->by_ipt = FastDiv::make(plan->iters_per_tile);
  dp->by_tiles_n = FastDiv::make(plan->num_block_n);
  dp->by_width = FastDiv::make((uint32_t)raster * plan->num_block_n);
  dp->by_raster = FastDiv::make(raster);
  dp->by_tail = FastDiv::make(dp->raster_tail);
  dp->by_full1 = FastDiv::make(plan->streamk_full_tiles + 1);
  dp->by_full = FastDiv::make(plan->streamk_full_tiles > 0 ? plan->streamk_full_tiles : 1);
  w->status = nullptr; w->flags = nullptr; w->partials = nullptr;
  if (plan->workspace_bytes > 0) {
    char *base = static_cast<char *>(ws);
    w->status = reinterpret_cast<int *>(base);
    w->flags = reinterpret_cast<int *>(base + 256);
    w->partials = reinterpret_cast<float *>(base + WS_PART_OFF);
  }
  (void)k;
  return SK_OK;
}

// family: 0 tile kernels, 1 small-M kernels, 2 fp32 kernels
int cached_occupancy(int id, int family) {
  static int cache[512];
  static bool have[512];
  const int slot = id & 511;  // kernel ids stay below 512
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!have[slot]) {
    cache[slot] = family == 1 ? occupancy_skinny(id) : (family == 2 ? occupancy_f32(id) : occupancy_tile(id));
    have[slot] = true;
  }
  return cache[slot];
}

}  // namespace

extern "C" int sk_version(void) { return SK_VERSION; }

extern "C" const char *sk_kernel_name(int kernel_id) {
  const KernelInfo *k = kernel_by_id(kernel_id);
  return k ? k->name : nullptr;
}

extern "C" const char *sk_strerror(int s) {
  switch (s) {
    case SK_OK: return "ok";
    case SK_ERR_NULL: return "null pointer";
    case SK_ERR_SHAPE: return "bad shape or leading dimension";
    case SK_ERR_ALIGN: return "misaligned pointer, leading dimension or K";
    case SK_ERR_CONFIG: return "unsupported tile / grid / schedule / fix-up, or plan does not match the call";
    case SK_ERR_WORKSPACE: return "workspace missing or too small";
    case SK_ERR_LAUNCH: return "HIP launch failed";
    case SK_ERR_DEVICE: return "no usable gfx950 device";
    case SK_ERR_TIMEOUT: return "fix-up wait timed out; re-initialise the workspace";
  }
  return "unknown status";
}

extern "C" int sk_device_info(int *num_cus, int *clock_khz, int *lds_bytes_per_cu) {
  const DeviceInfo d = device_info();
  if (!d.ok) return SK_ERR_DEVICE;
  if (num_cus) *num_cus = d.cus;
  if (clock_khz) *clock_khz = d.clock_khz;
  if (lds_bytes_per_cu) *lds_bytes_per_cu = d.lds;
  return SK_OK;
}

extern "C" int sk_workspace_init(void *ws, size_t ws_bytes, void *stream) {
  if (ws_bytes == 0) return SK_OK;
  if (!ws) return SK_ERR_NULL;
  if ((reinterpret_cast<uintptr_t>(ws) & 3) || (ws_bytes & 3)) return SK_ERR_ALIGN;
  const size_t n = ws_bytes / 4;
  int blocks = (int)((n + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                     static_cast<uint32_t *>(ws), n);
  if (hipGetLastError() != hipSuccess) return SK_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_mutex);
  g_ws[ws] = WsInfo{ws_bytes, false};
  return SK_OK;
}

extern "C" int sk_workspace_release(void *ws) {
  if (!ws) return SK_ERR_NULL;
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_ws.erase(ws) ? SK_OK : SK_ERR_WORKSPACE;
}

extern "C" int sk_workspace_status(void *ws, void *stream) {
  if (!ws) return SK_ERR_NULL;
  int v = 0;
  if (hipMemcpyAsync(&v, ws, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess)
    return SK_ERR_LAUNCH;
  if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return SK_ERR_LAUNCH;
  if (v == 0) return SK_OK;
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_ws.find(ws);
  if (it != g_ws.end()) it->second.poisoned = true;
  return SK_ERR_TIMEOUT;
}

// checks an sk_epilogue and packs it into the one word the kernels take (0 = no epilogue)
static int epilogue_word(const sk_epilogue *epi, const void **word) {
  *word = nullptr;
  if (!epi) return SK_OK;
  if (epi->reserved[0] || epi->reserved[1]) return SK_ERR_CONFIG;
  if (epi->activation < SK_ACT_NONE || epi->activation > SK_ACT_SILU) return SK_ERR_CONFIG;
  const uintptr_t b = reinterpret_cast<uintptr_t>(epi->bias);
  if (b & 1) return SK_ERR_ALIGN;
  if (b >> EPI_ACT_SHIFT) return SK_ERR_CONFIG;  // not a device address
  *word = epi_word(epi->bias, (int)epi->activation);
  return SK_OK;
}

static int gemm_16bit(int dtype, const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                      int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                      size_t ws_bytes, void *stream, const sk_epilogue *epi = nullptr, bool is_static = false) {
  const void *bias = nullptr;  // the kernels' epilogue word: bias pointer and activation code
  if (int rc = epilogue_word(epi, &bias)) return rc;
  if (!A || !B || !C) return SK_ERR_NULL;
  int rc = check_plan(plan, M, N, K, dtype, plan ? plan->layout : 0);
  if (rc) return rc;
  const bool nn = plan->layout == SK_LAYOUT_NN;
  if (lda < K || ldb < (nn ? N : K) || ldc < N) return SK_ERR_SHAPE;
  if ((K % 8) || (lda % 8) || (ldb % 8) || (nn && (N % 8))) return SK_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(B) & 15) ||
      (reinterpret_cast<uintptr_t>(C) & 1))
    return SK_ERR_ALIGN;
  const KernelInfo *k = kernel_by_id(plan->kernel_id);
  if (!k || k->dtype != dtype || k->layout != plan->layout) return SK_ERR_CONFIG;
  // a tile's rows (NN: all K rows of B) must be addressable with 32-bit byte offsets
  if (lda * 2 * k->bm >= (int64_t)1 << 31 || ldb * 2 * (nn ? K : k->bn) >= (int64_t)1 << 31) return SK_ERR_SHAPE;
  DevPlan dp;
  Workspace w;
  const bool skinny = k->family == FAMILY_SKINNY;
  if (plan->fixup == SK_FIXUP_ATOMIC_C && plan->streamk_tiles > 0) {
    // partial tiles are added into C itself, two elements per atomic: C starts at zero, pairs must be aligned,
    // and there is no CTA that would apply a bias once
    if (bias != nullptr || skinny) return SK_ERR_CONFIG;
    if ((N % 2) || (ldc % 2) || (reinterpret_cast<uintptr_t>(C) & 3)) return SK_ERR_ALIGN;
  }
  rc = make_dev_plan(plan, k, ws, ws_bytes, cached_occupancy(k->id, skinny ? 1 : 0), (hipStream_t)stream, &dp, &w,
                     is_static);
  if (rc) return rc;
  if (plan->fixup == SK_FIXUP_ATOMIC_C && plan->streamk_tiles > 0) {
    // (behind every check: a call that is refused leaves the caller's C alone)
    hipLaunchKernelGGL(zero_pairs_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<uint32_t *>(C),
                       (int)M, (int)(N / 2), (int64_t)(ldc / 2));
    if (hipGetLastError() != hipSuccess) return SK_ERR_LAUNCH;
  }
  int herr;
  if (skinny) {
    SkinnyArgs a{(const half_t *)A, B, nullptr, (half_t *)C, (int)M, (int)N, (int)K, lda, ldb, ldc, 0, 0, nullptr};
    herr = launch_skinny(k->id, a, dp, w, (hipStream_t)stream, bias);
  } else {
    GemmArgs a{(const half_t *)A, (const half_t *)B, (half_t *)C, (int)M, (int)N, (int)K, lda, ldb, ldc, 1.f};
    herr = launch_tile_f16(k->id, a, dp, w, (hipStream_t)stream, bias);
  }
  return herr == 0 ? SK_OK : SK_ERR_LAUNCH;
}

extern "C" int sk_gemm_f16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                           size_t ws_bytes, void *stream) {
  return gemm_16bit(SK_F16, A, B, C, M, N, K, lda, ldb, ldc, plan, ws, ws_bytes, stream);
}

extern "C" int sk_static_init(void) {
  void *ws = nullptr;
  return static_scratch(&ws);
}

extern "C" int sk_gemm_f16_static(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                                  int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *stream) {
  if (!plan) return SK_ERR_NULL;
  if ((uint64_t)plan->workspace_bytes > (uint64_t)SK_STATIC_WORKSPACE_BYTES) return SK_ERR_WORKSPACE;
  void *ws = nullptr;
  if (plan->workspace_bytes > 0)
    if (int rc = static_scratch(&ws)) return rc;
  return gemm_16bit(SK_F16, A, B, C, M, N, K, lda, ldb, ldc, plan, ws, ws ? (size_t)SK_STATIC_WORKSPACE_BYTES : 0, stream,
                    nullptr, true);
}

extern "C" int sk_gemm_f16_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                              size_t ws_bytes, void *stream, const sk_epilogue *epi) {
  return gemm_16bit(SK_F16, A, B, C, M, N, K, lda, ldb, ldc, plan, ws, ws_bytes, stream, epi);
}
extern "C" int sk_gemm_bf16_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                               size_t ws_bytes, void *stream, const sk_epilogue *epi) {
  return gemm_16bit(SK_BF16, A, B, C, M, N, K, lda, ldb, ldc, plan, ws, ws_bytes, stream, epi);
}

// bfloat16 kernels take the same 16-bit containers; only the MFMA and the rounding of C differ
extern "C" int sk_gemm_bf16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                            size_t ws_bytes, void *stream) {
  return gemm_16bit(SK_BF16, A, B, C, M, N, K, lda, ldb, ldc, plan, ws, ws_bytes, stream);
}

// one-byte operands (fp8, int8) travel through the fp16 tile machinery as pairs: K and the leading
// dimensions of A and B are handed to the kernel in 16-bit units
static int gemm_8bit(int dtype, const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                     int64_t lda, int64_t ldb, int64_t ldc, float alpha, const sk_plan *plan, void *ws,
                     size_t ws_bytes, void *stream, const sk_epilogue *epi = nullptr) {
  const void *bias = nullptr;  // the kernels' epilogue word (fp8 only: the int8 kernels store int32 sums)
  if (int rc = epilogue_word(epi, &bias)) return rc;
  if (!A || !B || !C) return SK_ERR_NULL;
  int rc = check_plan(plan, M, N, K, dtype, SK_LAYOUT_NT);
  if (rc) return rc;
  if (lda < K || ldb < K || ldc < N) return SK_ERR_SHAPE;
  if ((K % 16) || (lda % 16) || (ldb % 16)) return SK_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(B) & 15) ||
      (reinterpret_cast<uintptr_t>(C) & (dtype == SK_I8 ? 3 : 1)))
    return SK_ERR_ALIGN;
  const KernelInfo *k = kernel_by_id(plan->kernel_id);
  if (!k || k->dtype != dtype) return SK_ERR_CONFIG;
  if (lda * k->bm >= (int64_t)1 << 31 || ldb * k->bn >= (int64_t)1 << 31) return SK_ERR_SHAPE;
  DevPlan dp;
  Workspace w;
  const bool skinny = k->family == FAMILY_SKINNY;
  rc = make_dev_plan(plan, k, ws, ws_bytes, cached_occupancy(k->id, skinny ? 1 : 0), (hipStream_t)stream, &dp, &w);
  if (rc) return rc;
  if (skinny) {  // small-M fp8 / int8 kernels: bytes travel as pairs, alpha in the `zero` field (int8: C is int32)
    SkinnyArgs a{(const half_t *)A, B, nullptr, (half_t *)C, (int)M, (int)N, (int)(K / 2), lda / 2, ldb / 2, ldc,
                 __builtin_bit_cast(int, alpha), 0, nullptr};
    return launch_skinny(k->id, a, dp, w, (hipStream_t)stream, bias) == 0 ? SK_OK : SK_ERR_LAUNCH;
  }
  GemmArgs a{(const half_t *)A, (const half_t *)B, (half_t *)C, (int)M, (int)N, (int)(K / 2), lda / 2, ldb / 2, ldc, alpha};
  return launch_tile_f16(k->id, a, dp, w, (hipStream_t)stream, bias) == 0 ? SK_OK : SK_ERR_LAUNCH;
}

extern "C" int sk_gemm_f8(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc, float alpha, const sk_plan *plan, void *ws,
                          size_t ws_bytes, void *stream) {
  if (!(alpha == alpha) || alpha - alpha != 0.f) return SK_ERR_CONFIG;  // NaN or infinite
  const int dtype = plan && plan->dtype == SK_F8E5M2 ? SK_F8E5M2 : SK_F8E4M3;  // which format the bytes are in
  return gemm_8bit(dtype, A, B, C, M, N, K, lda, ldb, ldc, alpha, plan, ws, ws_bytes, stream);
}

extern "C" int sk_gemm_f8_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                             int64_t lda, int64_t ldb, int64_t ldc, float alpha, const sk_plan *plan, void *ws,
                             size_t ws_bytes, void *stream, const sk_epilogue *epi) {
  if (!(alpha == alpha) || alpha - alpha != 0.f) return SK_ERR_CONFIG;
  const int dtype = plan && plan->dtype == SK_F8E5M2 ? SK_F8E5M2 : SK_F8E4M3;
  return gemm_8bit(dtype, A, B, C, M, N, K, lda, ldb, ldc, alpha, plan, ws, ws_bytes, stream, epi);
}

// (C and ldc are int32 here; the kernel casts)
extern "C" int sk_gemm_i8(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                          size_t ws_bytes, void *stream) {
  return gemm_8bit(SK_I8, A, B, C, M, N, K, lda, ldb, ldc, 1.f, plan, ws, ws_bytes, stream);
}

extern "C" int sk_gemm_f32(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws,
                           size_t ws_bytes, void *stream) {
  if (!A || !B || !C) return SK_ERR_NULL;
  int rc = check_plan(plan, M, N, K, SK_F32, plan ? plan->layout : 0);
  if (rc) return rc;
  const bool nn = plan->layout == SK_LAYOUT_NN;
  if (lda < K || ldb < (nn ? N : K) || ldc < N) return SK_ERR_SHAPE;
  if ((K % 4) || (lda % 4) || (ldb % 4) || (nn && (N % 4))) return SK_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(B) & 15) ||
      (reinterpret_cast<uintptr_t>(C) & 3))
    return SK_ERR_ALIGN;
  const KernelInfo *k = kernel_by_id(plan->kernel_id);
  if (!k || k->dtype != SK_F32 || k->layout != plan->layout) return SK_ERR_CONFIG;
  if (lda * 4 * k->bm >= (int64_t)1 << 31 || ldb * 4 * (nn ? K : k->bn) >= (int64_t)1 << 31) return SK_ERR_SHAPE;
  DevPlan dp;
  Workspace w;
  rc = make_dev_plan(plan, k, ws, ws_bytes, cached_occupancy(k->id, 2), (hipStream_t)stream, &dp, &w);
  if (rc) return rc;
  GemmArgsF32 a{(const float *)A, (const float *)B, (float *)C, (int)M, (int)N, (int)K, lda, ldb, ldc};
  return launch_f32(k->id, a, dp, w, (hipStream_t)stream) == 0 ? SK_OK : SK_ERR_LAUNCH;
}

static int gemm_q4_any(const void *A, const void *Wq, const void *scales, const void *zeros, void *C, int64_t M,
                       int64_t N, int64_t K, int64_t lda, int64_t ldc, int group, int zero, int dtype,
                       const sk_plan *plan, void *ws, size_t ws_bytes, void *stream,
                       const sk_epilogue *epi = nullptr) {
  const void *bias = nullptr;  // the kernels' epilogue word: bias pointer and activation code
  if (int rc = epilogue_word(epi, &bias)) return rc;
  if (!A || !Wq || !scales || !C || ((dtype == SK_Q4_ZP || dtype == SK_Q4_ZP_TILED) && !zeros)) return SK_ERR_NULL;
  int rc = check_plan(plan, M, N, K, dtype, SK_LAYOUT_NT);
  if (rc) return rc;
  if (group != 128 || zero < 0 || zero > 15) return SK_ERR_CONFIG;
  if (lda < K || ldc < N) return SK_ERR_SHAPE;
  if ((K % 128) || (lda % 8)) return SK_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(Wq) & 15) ||
      (reinterpret_cast<uintptr_t>(scales) & 1) || (reinterpret_cast<uintptr_t>(zeros) & 1) ||
      (reinterpret_cast<uintptr_t>(C) & 1))
    return SK_ERR_ALIGN;
  const KernelInfo *k = kernel_by_id(plan->kernel_id);
  if (!k || k->dtype != dtype) return SK_ERR_CONFIG;
  if (lda * 2 * k->bm >= (int64_t)1 << 31 || (K / 2) * k->bn >= (int64_t)1 << 31) return SK_ERR_SHAPE;
  DevPlan dp;
  Workspace w;
  if (k->family == FAMILY_TILE) {
    // more than 64 rows of A: the tile kernels that dequantise B on its way into LDS (scalar zero point,
    // row-major nibbles)
    if (dtype != SK_Q4) return SK_ERR_CONFIG;
    rc = make_dev_plan(plan, k, ws, ws_bytes, cached_occupancy(k->id, 0), (hipStream_t)stream, &dp, &w);
    if (rc) return rc;
    GemmArgs g{(const half_t *)A, (const half_t *)Wq, (half_t *)C, (int)M, (int)N, (int)K, lda, K / 2, ldc, 1.f,
               (const half_t *)scales, zero, (int)(K / group)};
    return launch_tile_f16(k->id, g, dp, w, (hipStream_t)stream, bias) == 0 ? SK_OK : SK_ERR_LAUNCH;
  }
  if (k->family != FAMILY_SKINNY) return SK_ERR_CONFIG;
  rc = make_dev_plan(plan, k, ws, ws_bytes, cached_occupancy(k->id, 1), (hipStream_t)stream, &dp, &w);
  if (rc) return rc;
  SkinnyArgs a{(const half_t *)A, Wq, (const half_t *)scales, (half_t *)C, (int)M, (int)N, (int)K,
               lda, K / 2, ldc, zero, (int)(K / group), (const half_t *)zeros};
  int herr = launch_skinny(k->id, a, dp, w, (hipStream_t)stream, bias);
  return herr == 0 ? SK_OK : SK_ERR_LAUNCH;
}

extern "C" int sk_gemm_q4(const void *A, const void *Wq, const void *scales, void *C, int64_t M, int64_t N,
                          int64_t K, int64_t lda, int64_t ldc, int group, int zero, const sk_plan *plan,
                          void *ws, size_t ws_bytes, void *stream) {
  const int dtype = plan && plan->dtype == SK_Q4_TILED ? SK_Q4_TILED : SK_Q4;  // which layout Wq is in
  return gemm_q4_any(A, Wq, scales, nullptr, C, M, N, K, lda, ldc, group, zero, dtype, plan, ws, ws_bytes, stream);
}

extern "C" int sk_gemm_q4_ex(const void *A, const void *Wq, const void *scales, const void *zeros, void *C,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc, int group, int zero,
                             const sk_plan *plan, void *ws, size_t ws_bytes, void *stream, const sk_epilogue *epi) {
  const int dtype = zeros ? (plan && plan->dtype == SK_Q4_ZP_TILED ? SK_Q4_ZP_TILED : SK_Q4_ZP)
                          : (plan && plan->dtype == SK_Q4_TILED ? SK_Q4_TILED : SK_Q4);
  return gemm_q4_any(A, Wq, scales, zeros, C, M, N, K, lda, ldc, group, zeros ? 0 : zero, dtype, plan, ws, ws_bytes,
                     stream, epi);
}

extern "C" int sk_gemm_q4_zp(const void *A, const void *Wq, const void *scales, const void *zeros, void *C,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc, int group,
                             const sk_plan *plan, void *ws, size_t ws_bytes, void *stream) {
  const int dtype = plan && plan->dtype == SK_Q4_ZP_TILED ? SK_Q4_ZP_TILED : SK_Q4_ZP;  // which layout Wq is in
  return gemm_q4_any(A, Wq, scales, zeros, C, M, N, K, lda, ldc, group, 0, dtype, plan, ws, ws_bytes, stream);
}

namespace {
// one thread per 32-bit word of packed nibbles: 8 weights, written in natural element order
__global__ void dequant_q4_kernel(const uint32_t *wq, const half_t *scales, const half_t *zeros, half_t *out,
                                  int64_t words, int words_per_row, int groups, int group, int zero) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= words) return;
  const int64_t row = i / words_per_row;
  const int k = (int)(i % words_per_row) * 8;
  const half_t s = scales[row * groups + k / group];
  half8v v;
  if (zeros) {  // one zero point per group and row
    const half_t z = zeros[row * groups + k / group];
    const half_t lo = (half_t)1024.f + z, hi = (half_t)-64.f - z;
    v = dequant_word_q4(wq[i], q4_consts(0), half2v{s, s}, half2v{lo, lo}, half2v{hi, hi});
  } else {
    v = dequant_word_q4(wq[i], q4_consts(zero), half2v{s, s});
  }
  half8v o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = v[q4_slot_of_element(e)];
  *reinterpret_cast<half8v *>(out + i * 8) = o;
}
}  // namespace

static int dequant_q4_any(const void *Wq, const void *scales, const void *zeros, void *W, int64_t N, int64_t K,
                          int group, int zero, void *stream);
extern "C" int sk_dequant_q4(const void *Wq, const void *scales, void *W, int64_t N, int64_t K, int group,
                             int zero, void *stream) {
  return dequant_q4_any(Wq, scales, nullptr, W, N, K, group, zero, stream);
}
extern "C" int sk_dequant_q4_zp(const void *Wq, const void *scales, const void *zeros, void *W, int64_t N,
                                int64_t K, int group, void *stream) {
  if (!zeros) return SK_ERR_NULL;
  return dequant_q4_any(Wq, scales, zeros, W, N, K, group, 0, stream);
}
static int dequant_q4_any(const void *Wq, const void *scales, const void *zeros, void *W, int64_t N, int64_t K,
                          int group, int zero, void *stream) {
  if (!Wq || !scales || !W) return SK_ERR_NULL;
  if (N <= 0 || K <= 0) return SK_ERR_SHAPE;
  if (group <= 0 || (group % 8) || (K % group) || zero < 0 || zero > 15) return SK_ERR_CONFIG;
  if ((reinterpret_cast<uintptr_t>(Wq) & 3) || (reinterpret_cast<uintptr_t>(W) & 15)) return SK_ERR_ALIGN;
  const int64_t words = N * K / 8;
  const int64_t blocks = (words + 255) / 256;
  if (blocks > 0x7fffffff) return SK_ERR_SHAPE;
  hipLaunchKernelGGL(dequant_q4_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t *)Wq, (const half_t *)scales, (const half_t *)zeros, (half_t *)W, words,
                     (int)(K / 8), (int)(K / group), group, zero);
  return hipGetLastError() == hipSuccess ? SK_OK : SK_ERR_LAUNCH;
}
