// Device-side pieces shared by every Stream-K kernel: the plan as the kernels see it, the
// CTA -> work mapping, and the two partial-tile fix-ups.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace sk {

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

enum { FIXUP_ATOMIC = 1, FIXUP_REDUCE = 2, FIXUP_ATOMIC_C = 3 };

// Division of a non-negative 32-bit integer by a divisor known on the host: the host stores
// mul = floor(2^32 (2^shift - d) / d) + 1 with shift = ceil(log2 d), and
// n / d == (umulhi(n, mul) + n) >> shift for every 0 <= n < 2^31.  The kernels divide wave-uniform
// values only, so this is a handful of scalar instructions instead of a reciprocal sequence.
struct FastDiv {
  uint32_t mul, shift;
#if defined(__HIPCC__)
  __device__ __forceinline__ int div(int n) const { return (int)((__umulhi((uint32_t)n, mul) + (uint32_t)n) >> shift); }
#endif
  static FastDiv make(uint32_t d) {
    FastDiv f{1u, 0u};
    if (d <= 1) return f;
    while ((1ull << f.shift) < d) ++f.shift;
    f.mul = (uint32_t)((((1ull << f.shift) - d) << 32) / d + 1);
    return f;
  }
};

// A loop over [I0, I1) whose counter is a compile-time constant inside the body (f receives
// std::integral_constant<int, I>).  For loops that index the accumulator arrays and are too large for
// the unroller's size limit: a dynamic index would keep the accumulators in scratch memory.
template <int I0, int I1, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I0 < I1) {
    f(std::integral_constant<int, I0>{});
    static_for<I0 + 1, I1>(f);
  }
}

struct DevPlan {
  int tiles_m, tiles_n, ipt;  // tile grid, K-iterations per tile
  int total_tiles, sk_tiles;  // Stream-K tiles are ids [0, sk_tiles)
  int sk_full, sk_extra;      // iterations per CTA / CTAs that get one more
  int grid;                   // persistent CTAs
  int fixup;                  // FIXUP_ATOMIC, FIXUP_REDUCE or FIXUP_ATOMIC_C
  int raster;                 // 0 row-major, g > 0 grouped by g tile rows
  int spin_limit;             // polls before a waiting owner gives up
  int xcd_remap;              // 1: spread logical CTA ids so each XCD owns a contiguous range
  int raster_tail;            // tile rows in the last raster group (tiles_m % raster, or raster)
  int halves;                 // REDUCE plan whose every Stream-K tile is cut into two (1) or four (2) equal CTA segments
  int partials16;             // such a plan exchanges its half tiles rounded to C's 16-bit type (SK_FIXUP_REDUCE16)
  int perm_s, perm_g;         // perm_s > 1: Stream-K tile v stands at position (v % perm_s) * perm_g + v / perm_s
  FastDiv by_ipt, by_tiles_n, by_width, by_raster, by_tail, by_full1, by_full, by_perm;
};

// Words of the workspace's status block: WS_STATUS a timed-out fix-up wait (0 or SK_ERR_TIMEOUT),
// WS_DIRTY how far the partial area holds leftovers of REDUCE launches (256-byte units from its
// start), WS_CLEAN_DONE the block counter of the kernel that zero-fills it again.
enum { WS_STATUS = 0, WS_DIRTY = 1, WS_CLEAN_DONE = 2 };

struct Workspace {
  int *status;
  int *flags;
  float *partials;
};

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Giving XCD x a contiguous range of
// logical ids makes neighbouring tiles share an L2: XCD x runs the grid/8 workgroups b = x, x + 8, ... (one more
// on the first grid % 8 XCDs), and they get the ids from x * (grid / 8) + min(x, grid % 8) on.
__device__ __forceinline__ int logical_pid(const DevPlan &p) {
  const int b = blockIdx.x;
  if (p.xcd_remap) {
    const int x = b & 7;
    return x * (p.grid >> 3) + min(x, p.grid & 7) + (b >> 3);
  }
  return b;
}

__device__ __forceinline__ void sk_range(const DevPlan &p, int pid, int &start, int &last) {
  start = pid * p.sk_full + min(pid, p.sk_extra);
  last = (pid + 1) * p.sk_full + min(pid + 1, p.sk_extra);
}

__device__ __forceinline__ void tile_coords(const DevPlan &p, int tile, int &pm, int &pn) {
  if (p.perm_s > 1 && tile < p.sk_tiles) {  // interleaved order of the Stream-K tiles (sk_plan.interleave)
    const int q = p.by_perm.div(tile);
    tile = (tile - q * p.perm_s) * p.perm_g + q;
  }
  if (p.tiles_m == 1) {
    pm = 0;
    pn = tile;
  } else if (p.raster <= 0) {
    pm = p.by_tiles_n.div(tile);
    pn = tile - pm * p.tiles_n;
  } else {
    const int width = p.raster * p.tiles_n;
    const int group = p.by_width.div(tile);
    const int first_m = group * p.raster;
    const int r = tile - group * width;
    const bool tail = first_m + p.raster > p.tiles_m;
    const int gsize = tail ? p.raster_tail : p.raster;
    pn = tail ? p.by_tail.div(r) : p.by_raster.div(r);
    pm = first_m + r - pn * gsize;
  }
}

// ---- coherent workspace access ----
// Partial tiles and flags travel between CTAs on different XCDs, each with its own L2.  Every
// access to them is a device-scope relaxed atomic (64 bits at most), which the hardware performs
// coherently (write-through stores, loads that never return a stale L2 line).  That keeps the
// fix-up free of whole-L2 write-back / invalidate operations, which cost far more than the few
// kilobytes exchanged here and would be paid by every CTA.
__device__ __forceinline__ void st_coherent(float *p, floatx4 v) {
  union { floatx4 f; uint64_t u[2]; } c;
  c.f = v;
  __hip_atomic_store(reinterpret_cast<uint64_t *>(p), c.u[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(reinterpret_cast<uint64_t *>(p) + 1, c.u[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ floatx4 ld_coherent(const float *p) {
  union { floatx4 f; uint64_t u[2]; } c;
  c.u[0] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  c.u[1] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return c.f;
}
// the same for int32 accumulators (kept in integer registers from the MFMA to memory)
typedef int intx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st_coherent(int *p, intx4_t v) {
  union { intx4_t i; uint64_t u[2]; } c;
  c.i = v;
  __hip_atomic_store(reinterpret_cast<uint64_t *>(p), c.u[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(reinterpret_cast<uint64_t *>(p) + 1, c.u[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ intx4_t ld_coherent(const int *p) {
  union { intx4_t i; uint64_t u[2]; } c;
  c.u[0] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  c.u[1] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return c.i;
}
__device__ __forceinline__ void st_coherent(int *p, int v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ld_coherent_scalar(const int *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_coherent(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_coherent_scalar(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Every vector memory operation this thread has issued -- loads, stores and atomics without return all
// count on vmcnt on this target -- has been acknowledged by the memory system.  A workgroup-scope
// fence is not enough: it waits for LDS traffic only, and the barrier that follows adds no wait of
// its own, so a flag raised after it could overtake the partial it announces.
__device__ __forceinline__ void wait_own_memory_ops() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---- REDUCE fix-up: flags ----
// Contributor: every thread waits for its own (write-through) partial stores, the barrier
// collects the CTA, then thread 0 raises the flag.
// COHERENT = false: the partial went through the L2 with ordinary stores; thread 0's device-scope
// release (one L2 write-back for the whole CTA, after the barrier has collected everybody's
// stores) publishes it together with the flag.
// dirty_mark / dirty_units: the workspace's record of how far its partial area holds leftovers
// (256-byte units) is raised past this CTA's slot, for the launch that next needs the area zeroed.
template <bool COHERENT>
__device__ __forceinline__ void signal_partial_ready(int *flag, int *dirty_mark, int dirty_units) {
  wait_own_memory_ops();
  __syncthreads();
  if (threadIdx.x == 0) {
    __hip_atomic_fetch_max(dirty_mark, dirty_units, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (COHERENT)
      __hip_atomic_store(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
      __hip_atomic_store(flag, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// CTA that owns K-iteration `iter` of the Stream-K wave (inverse of sk_range)
__device__ __forceinline__ int sk_pid_of_iter(const DevPlan &p, int iter) {
  const int boundary = p.sk_extra * (p.sk_full + 1);
  if (iter < boundary) return p.by_full1.div(iter);
  return p.sk_extra + p.by_full.div(iter - boundary);
}

// Owner: the first wave polls all `npeers` follower flags at once, one flag per lane; the barrier
// orders the CTA's (coherent) partial loads after the flags were seen.
// Returns false if the poll limit ran out.
// COHERENT = false: one device-scope acquire (L2 invalidate) by the polling wave before the
// barrier, so that the ordinary loads that follow cannot hit stale lines.
// WORD: lds_word is a word of LDS of the caller's through which the first wave's result reaches the others; without one
// the device library's block-wide AND does it, which reserves 256 bytes of LDS of its own.
template <bool COHERENT, bool WORD = false>
__device__ __forceinline__ bool wait_partials_ready(int *flags, int npeers, int spin_limit, int *lds_word = nullptr) {
  int ok = 1;
  if (threadIdx.x < 64) {
    for (int i = threadIdx.x; i < npeers; i += 64) {
      int got = 0;
      for (int s = 0; s < spin_limit; ++s) {
        if (__hip_atomic_load(flags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { got = 1; break; }
        __builtin_amdgcn_s_sleep(1);
      }
      ok &= got;
    }
    if (!COHERENT) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  if constexpr (!WORD) {
    return __syncthreads_and(ok) != 0;
  } else {
    if (threadIdx.x < 64) {
      const bool all = __builtin_amdgcn_ballot_w64(ok == 0) == 0;
      if (threadIdx.x == 0) *lds_word = all;
    }
    __syncthreads();
    const bool all = *lds_word != 0;
    __syncthreads();
    return all;
  }
}

__device__ __forceinline__ void clear_flags_after_use(int *flags, int npeers) {
  __syncthreads();
  for (int i = threadIdx.x; i < npeers; i += blockDim.x)
    __hip_atomic_store(flags + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- buffer addressing ----
// A 128-bit buffer descriptor gives hardware range checking: a load whose byte offset is at or past
// num_bytes returns zeros.  Tiles hanging over the matrix edge need no predication, and a K tail
// is masked by pushing the per-lane offset out of range.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
__device__ __forceinline__ BufferRsrc make_rsrc(const void *base, uint32_t num_bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)num_bytes, 0x00020000);
}
__device__ __forceinline__ uint4v buffer_load_16(BufferRsrc r, uint32_t lane_off, uint32_t uniform_off) {
  return __builtin_bit_cast(uint4v, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, uniform_off, 0));
}
constexpr uint32_t OOB_OFFSET = 0x80000000u;

// 16-byte accesses of device scope (the sc1 bit: stores write through to memory, loads never return
// a line another XCD's L2 has since overwritten) -- the full-width form of st_coherent / ld_coherent
// for partial tiles of hundreds of KB.  off = per-lane byte offset, uoff = wave-uniform byte offset.
constexpr int CACHE_POLICY_SC1 = 16;
__device__ __forceinline__ void st_coherent16(BufferRsrc r, uint32_t off, uint32_t uoff, uint4v v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, off, uoff, CACHE_POLICY_SC1);
}
__device__ __forceinline__ uint4v ld_coherent16(BufferRsrc r, uint32_t off, uint32_t uoff) {
  return __builtin_bit_cast(uint4v, __builtin_amdgcn_raw_buffer_load_b128(r, off, uoff, CACHE_POLICY_SC1));
}

// Direct global -> LDS load, 16 bytes per lane: lane l's data lands at lds_base + 16*l.  Issued as
// inline assembly on purpose: the compiler's wait-count insertion cannot tell which LDS stage an
// in-flight load writes and would otherwise stall every LDS read on all of them.  The kernels
// that use this wait (vmcnt) and barrier by hand.  lds_base, rsrc and uniform_off are
// wave-uniform.
__device__ __forceinline__ uint4v make_rsrc_words(const void *base, uint32_t num_bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  return uint4v{(uint32_t)b, (uint32_t)(b >> 32) & 0xffffu, num_bytes, 0x00020000u};
}
// a descriptor whose words the compiler holds in vector registers although they are wave-uniform (values derived
// from the wave's index): moved to scalar registers, which is where an instruction wants them
__device__ __forceinline__ uint4v uniform_rsrc(uint4v w) {
  return uint4v{(uint32_t)__builtin_amdgcn_readfirstlane((int)w[0]), (uint32_t)__builtin_amdgcn_readfirstlane((int)w[1]),
                (uint32_t)__builtin_amdgcn_readfirstlane((int)w[2]), (uint32_t)__builtin_amdgcn_readfirstlane((int)w[3])};
}
__device__ __forceinline__ void dma_load_16(uint4v rsrc, uint32_t lds_base, uint32_t lane_off,
                                            uint32_t uniform_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(lane_off), "s"(rsrc), "s"(uniform_off)
               : "memory", "m0");
}
// Kernels that stream weight rows in long contiguous pieces (tile_stream_pairs.h) start their CTAs together, and the
// pitch of the rows is a large power of two: walking every tile from K = 0 has all CTAs read the same K offset of
// their rows at the same moment, which the memory system serves badly (N = K = 8192 fp16, 16 rows of A: 33.3 us;
// 27.8 us when neighbouring tiles start one iteration apart; 24.6 us with the starts below).  Tile pn starts
// rot = (3 pn + pn / 16) % n iterations into its segment of n iterations and wraps around; iterations past the
// segment keep their number (their loads fetch nothing).  The sum of a tile is therefore added up in a K order that
// depends on the tile, the same on every launch.
__device__ __forceinline__ int rotation_of(int pn, int n) { return n > 0 ? (3 * pn + (pn >> 4)) % n : 0; }
__device__ __forceinline__ int rotated_iteration(int t, int rot, int n) {
  const int r = t + rot;
  return t >= n ? t : (r >= n ? r - n : r);
}
__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

// Makes a pointer opaque to the optimiser at this program point.  The fix-up paths address dozens
// of far-apart float4 slots per thread; without this the address arithmetic is hoisted out of the
// persistent loop and kept in registers across the MFMA main loop.
template <class T>
__device__ __forceinline__ T *pin_here(T *p) {
  asm volatile("" : "+v"(p));
  return p;
}

// the same for a lane-dependent integer (column arithmetic of an epilogue operand)
__device__ __forceinline__ int pin_here(int x) {
  asm volatile("" : "+v"(x));
  return x;
}

// The epilogue's kernel argument is one 64-bit word: the bias pointer in the low 60 bits (device addresses use 57 at
// most) and the activation code in the top four.  Zero means "no epilogue", so kernels test one value, and the word
// costs the kernels that predate the activation no further argument.
constexpr int EPI_ACT_SHIFT = 60;
__host__ __device__ __forceinline__ const void *epi_word(const void *bias, int act) {
  return reinterpret_cast<const void *>(reinterpret_cast<uintptr_t>(bias) | ((uintptr_t)(uint32_t)act << EPI_ACT_SHIFT));
}
__device__ __forceinline__ int epi_act(const void *word) {
  return (int)(reinterpret_cast<uintptr_t>(word) >> EPI_ACT_SHIFT);
}
__device__ __forceinline__ const half_t *epi_bias(const void *word) {
  return reinterpret_cast<const half_t *>(reinterpret_cast<uintptr_t>(word) & (((uintptr_t)1 << EPI_ACT_SHIFT) - 1));
}

// activation applied in fp32 after the bias, before the rounding to C's type; act is uniform over the grid
// (codes are sk_activation's: 1 relu, 2 gelu in its tanh form, 3 silu)
__device__ __forceinline__ float activate(float x, int act) {
  if (act == 1) return fmaxf(x, 0.f);
  if (act == 2) {
    // 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)),  u = sqrt(2/pi) (x + 0.044715 x^3)
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x / (1.f + __expf(-2.f * u));
  }
  if (act == 3) return x / (1.f + __expf(-x));
  return x;
}

// optional epilogue operand: a row vector added to every row of C in fp32, before the rounding to C's type
// (fp16 bits, or bfloat16 bits when BF16).  Returns 0 without a bias or past the last column.
template <bool BF16 = false>
__device__ __forceinline__ float bias_at(const half_t *bias, int col, int N) {
  if (bias == nullptr || col >= N) return 0.f;
  if constexpr (BF16) {
    const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, bias[col]) << 16;
    return __builtin_bit_cast(float, bits);
  } else {
    return (float)bias[col];
  }
}

// four consecutive bias values starting at column col (a multiple of 4): one 8-byte load where the row allows it
template <bool BF16 = false>
__device__ __forceinline__ floatx4 bias4_at(const half_t *bias, int col, int N) {
  floatx4 r = {0.f, 0.f, 0.f, 0.f};
  if (bias == nullptr) return r;  // an activation without a bias
  if (col + 4 <= N && (reinterpret_cast<uintptr_t>(bias) & 7) == 0) {
    const half4v h = *reinterpret_cast<const half4v *>(bias + col);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (BF16)
        r[e] = __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, (half_t)h[e]) << 16);
      else
        r[e] = (float)h[e];
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = bias_at<BF16>(bias, col + e, N);
  }
  return r;
}

__device__ __forceinline__ void atomic_add_f32(float *p, float v) {
  // hardware global_atomic_add_f32, no return value, device scope
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Two fp32 values, rounded to C's 16-bit type, added to two adjacent elements of C with one packed atomic
// (global_atomic_pk_add_f16 / _bf16; p 4-byte aligned): the reference's atomic_addx2, streamk_fp16.py:248-255
template <bool BF16>
__device__ __forceinline__ void atomic_add_pair16(half_t *p, float x0, float x1) {
  if constexpr (BF16) {
    typedef short short2v __attribute__((ext_vector_type(2)));
    const __bf16 b0 = (__bf16)x0, b1 = (__bf16)x1;
    const short2v v = {__builtin_bit_cast(short, b0), __builtin_bit_cast(short, b1)};
    __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) short2v *)p, v);
  } else {
    const half2v v = {(half_t)x0, (half_t)x1};
    __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) half2v *)p, v);
  }
}
__device__ __forceinline__ void atomic_add_i32(int *p, int v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace sk
