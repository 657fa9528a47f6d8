// Shared host/device helpers for libzen_hip (gfx950, wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "zen_hip.h"

namespace zen {

// ------------------------------------------------------------------ host side

extern thread_local char g_last_error[256];

inline int fail(int code, const char *what) {
  snprintf(g_last_error, sizeof(g_last_error), "%s", what);
  return code;
}

inline int hip_fail(hipError_t e, const char *where) {
  snprintf(g_last_error, sizeof(g_last_error), "%s: %s", where, hipGetErrorString(e));
  return ZEN_EHIP;
}

#define ZEN_HIP_CHECK(expr)                                      \
  do {                                                           \
    hipError_t zen_e_ = (expr);                                  \
    if (zen_e_ != hipSuccess) return ::zen::hip_fail(zen_e_, #expr); \
  } while (0)

#define ZEN_LAUNCH_CHECK(name)                                   \
  do {                                                           \
    hipError_t zen_e_ = hipGetLastError();                       \
    if (zen_e_ != hipSuccess) return ::zen::hip_fail(zen_e_, name); \
  } while (0)

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Carves 256-byte aligned sub-buffers out of one workspace.
struct Carver {
  char *base;
  size_t used = 0;
  explicit Carver(void *p) : base(static_cast<char *>(p)) {}
  template <typename T>
  T *take(size_t count) {
    T *p = reinterpret_cast<T *>(base + used);
    used += align_up(count * sizeof(T), 256);
    return p;
  }
};

inline int ceil_log2_u64(uint64_t x) {  // bits needed to represent values in [0, x]
  int b = 0;
  while (b < 64 && (x >> b) != 0) ++b;
  return b;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Kernel timing tags (zen_profile.hip).  A ProfScope around a launch records
// HIP events on the launch stream when profiling is enabled; otherwise it is
// one relaxed load of a flag and a branch.
enum ProfTag {
  kProfTopkHist = 0,
  kProfSelectCompact,
  kProfInsertList,
  kProfFinalKey,
  kProfSort,
  kProfGather,
  kProfMergePrep,
  kProfMergeReduce,
  kProfCompress,
  kProfInsertDense,
  kProfSelectStage,
  kProfFeed,
  kProfSlabSort,
  kProfSlabChains,
  kProfSlabPlace,
  kProfMergeFeed,
  kProfMergeBucket,
  kProfSampleHist,
  kProfDecodeFused,
  kProfWideTail,
  kProfWideScatter,
  kProfWideMerge,
  kProfCount
};

class ProfScope {
 public:
  ProfScope(int tag, hipStream_t stream);
  ~ProfScope();
  ProfScope(const ProfScope &) = delete;
  ProfScope &operator=(const ProfScope &) = delete;

 private:
  int tag_;
  hipStream_t stream_;
  hipEvent_t start_, stop_;
};

// ---------------------------------------------------------------- device side

constexpr uint32_t kSeed1 = 10001861u;  // functions_cuda_kernel.cu:101
constexpr uint32_t kSeed2 = 100703u;    // functions_cuda_kernel.cu:124
constexpr uint32_t kSeed3 = 5002639u;   // functions_cuda_kernel.cu:151

// functions_cuda_kernel.cu:80-88 without the additive seed, in Horner form
// (identical in uint32 ring arithmetic).  h(k, c) = poly(k) + c.
__host__ __device__ inline uint32_t poly(uint32_t k) {
  return ((573729859u * k + 0xcc9e2d51u) * k + 0x1b873593u) * k;
}

// Probe geometry of the hash table: level 0 probes the whole table, levels 1
// and 2 probe inside the partition level 0 landed in
// (functions_cuda_kernel.cu:101-107, 119-129, 144-156).
struct Probe {
  uint32_t m;    // table size
  uint32_t npp;  // slots per partition = m / partitions
  int levels;    // 1, 2 or 3
};

__device__ inline uint32_t probe_slot(const Probe &g, uint32_t t, int level, uint32_t *part_out) {
  const uint32_t h = poly(t);
  const uint32_t first = (h + kSeed1) % g.m;
  const uint32_t part = first / g.npp;
  *part_out = part;
  if (level == 0) return first;
  const uint32_t seed = level == 1 ? kSeed2 : kSeed3;
  return part * g.npp + (h + seed) % g.npp;
}

// Element storage and magnitude keys (bit pattern with the sign cleared).
template <typename S>
struct KeyOf;
template <>
struct KeyOf<uint16_t> {
  static constexpr uint32_t kMask = 0x7fffu;
  static constexpr int kBits = 15;
  static __device__ inline float to_f32(uint16_t v) { return __uint_as_float(uint32_t(v) << 16); }
};
template <>
struct KeyOf<uint32_t> {
  static constexpr uint32_t kMask = 0x7fffffffu;
  static constexpr int kBits = 31;
  static __device__ inline float to_f32(uint32_t v) { return __uint_as_float(v); }
};

__device__ inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}

// Waits until the global memory operations this wave has issued, stores and atomics without a return value
// included, have been acknowledged by the place that carries them out.
__device__ inline void wait_global_acks() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Reads a word that other workgroups of the running kernel have changed with device-wide atomics, from the
// place where those are carried out (not from this compute unit's caches).
__device__ inline uint32_t load_fresh(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ inline int lane_id() { return int(__lane_id()); }

__device__ inline uint64_t lanes_below() {  // mask of lanes with a smaller id
  return (1ull << lane_id()) - 1ull;
}

template <typename T>
__device__ inline T wave_inclusive_scan(T v) {
  const int lane = lane_id();
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    T o = __shfl_up(v, d, 64);
    if (lane >= d) v += o;
  }
  return v;
}

template <typename T>
__device__ inline T wave_sum(T v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}

// Exclusive scan over the threads of a block (BLOCK a multiple of 64).
// `total` receives the block sum in every thread.  smem needs BLOCK/64 + 1 T's.
template <typename T, int BLOCK>
__device__ inline T block_exclusive_scan(T v, T *smem, T *total) {
  constexpr int kWaves = BLOCK / 64;
  const int wave = threadIdx.x >> 6;
  const T incl = wave_inclusive_scan(v);
  if (lane_id() == 63) smem[wave] = incl;
  __syncthreads();
  T wave_base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const T s = smem[w];
    if (w < wave) wave_base += s;
    sum += s;
  }
  __syncthreads();
  *total = sum;
  return wave_base + incl - v;
}

// ------------------------------------------------ single-pass prefix over tiles
// Decoupled look-back.  One 64-bit descriptor per tile holds 2 flag bits and a
// 62-bit value, so flag and value are published by one atomic store: first the
// tile's own count (aggregate), later its inclusive prefix.  A tile sums the
// aggregates of its predecessors, 64 at a time, back to the nearest one that
// already shows a prefix.  Tiles take their id from a ticket counter, so every
// lower-numbered tile already runs and the wait cannot deadlock; it is also
// bounded.  The prefix frontier advances 64 tiles per memory round trip, so
// kernels keep their tile count in the low thousands.
//
// Scratch layout (all zero before the launch): ntiles descriptors and one
// ticket word = scan_words(ntiles) uint64.

constexpr uint64_t kDescAggregate = 1ull << 62;
constexpr uint64_t kDescPrefix = 2ull << 62;
constexpr uint64_t kDescValue = (1ull << 62) - 1;
constexpr uint32_t kSpinLimit = 1u << 22;  // bounded wait: flag ZEN_STAT_INTERNAL instead of hanging

constexpr size_t scan_words_c(int64_t ntiles) { return (size_t)ntiles + 2; }
inline size_t scan_words(int64_t ntiles) { return scan_words_c(ntiles); }

struct ScanState {
  unsigned long long *desc;
  uint32_t *ticket;
};

inline ScanState scan_state(void *scratch, int64_t ntiles) {
  ScanState st;
  st.desc = static_cast<unsigned long long *>(scratch);
  st.ticket = reinterpret_cast<uint32_t *>(st.desc + ntiles);
  return st;
}

__device__ inline uint64_t desc_load(const unsigned long long *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void desc_store(unsigned long long *p, uint64_t v) {
  __hip_atomic_store(p, (unsigned long long)v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every thread of the block.  Returns the sum of the aggregates of
// all tiles before `tile`.  smem: one uint64.
__device__ inline uint64_t lookback_exclusive(const ScanState &st, int tile, uint64_t aggregate,
                                              int32_t *status, uint64_t *smem) {
  unsigned long long *desc = st.desc;
  if (threadIdx.x < 64) {
    const int lane = lane_id();
    if (lane == 0) desc_store(&desc[tile], (tile == 0 ? kDescPrefix : kDescAggregate) | aggregate);
    uint64_t excl = 0;
    if (tile > 0) {
      int base = tile - 1;
      bool gave_up = false;
      for (;;) {
        const int p = base - lane;
        uint64_t d = kDescPrefix;  // tiles before the first: prefix 0
        if (p >= 0) {
          d = desc_load(&desc[p]);
          uint32_t spins = 0;
          while ((d >> 62) == 0) {
            if (++spins > kSpinLimit) {
              gave_up = true;
              d = kDescPrefix;
              break;
            }
            __builtin_amdgcn_s_sleep(2);
            d = desc_load(&desc[p]);
          }
        }
        const uint64_t have_prefix = __ballot((d >> 62) == 2);
        const int first = have_prefix ? __ffsll((unsigned long long)have_prefix) - 1 : 64;
        excl += wave_sum<uint64_t>(lane <= first ? (d & kDescValue) : 0ull);
        if (have_prefix) break;
        base -= 64;
      }
      if (gave_up) atomicOr(status, ZEN_STAT_INTERNAL);
      if (lane == 0) desc_store(&desc[tile], kDescPrefix | (excl + aggregate));
    }
    if (lane == 0) *smem = excl;
  }
  __syncthreads();
  const uint64_t r = *smem;
  __syncthreads();
  return r;
}

// Grid-stride fill; also the way to clear scratch without a memset node.
template <typename T>
__global__ void k_fill(T *p, T v, size_t count) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < count;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = v;
}

template <typename T>
inline void launch_fill(T *p, T v, size_t count, hipStream_t s) {
  if (count == 0) return;
  const size_t blocks = (count + 1023) / 1024;
  k_fill<T><<<dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, s>>>(p, v, count);
}

// ---------------------------------------------------------- sort (zen_sort.hip)

// Stable LSD radix sort of (key, val) pairs on the low `bits` bits.  The result
// ends in (keys_a, vals_a) when the returned value is 0 and in (keys_b,
// vals_b) when it is 1; negative = error.  `scratch` from sort_scratch_bytes.
// more_a / more_b: an optional second payload moved along with the first.
size_t sort_scratch_bytes(int64_t max_count);
int sort_pairs(uint32_t *keys_a, uint32_t *vals_a, uint32_t *keys_b, uint32_t *vals_b,
               int64_t max_count, const uint32_t *count_dev, int bits, void *scratch,
               int32_t *status, hipStream_t stream, uint32_t *more_a = nullptr, uint32_t *more_b = nullptr);

// Stable sort of records whose keys spread evenly over [0, sentinel) (hash slots, hashed indices): one
// scatter pass into 511 key ranges, then each range sorted inside LDS by one workgroup.  Records with
// key >= sentinel come last, in no particular order.  The result is in the b arrays (returns 1; negative =
// error).  A key range holding more records than fit in LDS sets ZEN_STAT_RETRY in *status and the order
// is then unspecified.  bucket_sort_fits: whether `expected` records (the live count may sit on the device)
// leave the key ranges room to spare; same scratch as sort_pairs.
bool bucket_sort_fits(int64_t expected, uint32_t sentinel);
int bucket_sort_pairs(uint32_t *keys_a, uint32_t *vals_a, uint32_t *keys_b, uint32_t *vals_b, int64_t max_count,
                      const uint32_t *count_dev, uint32_t sentinel, void *scratch, int32_t *status,
                      hipStream_t stream, uint32_t *more_a = nullptr, uint32_t *more_b = nullptr);

}  // namespace zen
