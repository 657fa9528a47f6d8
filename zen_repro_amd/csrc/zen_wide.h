// Wide buckets: the layout of the fast paths for inputs whose selected (or received) entries number a few
// million at most.
//
// The key space (level-1 hash slots on the encode side, indices on the merge side) is cut into at most 256
// contiguous key ranges, as many as the chip has compute units, and every bucket is handled by ONE workgroup
// of 1024 threads that has a compute unit's LDS to itself: up to kWideCap records are sorted there in one go
// (zen_slab.h needs a thousand buckets of a few thousand records for the same input, two rounds of workgroups
// and a scatter step of its own to feed them).  The producer appends its entries straight to the buckets: with
// 256 destinations a staged batch of a few thousand entries still leaves in runs of 8 to 16.
//
// A bucket's slab is kept in kWideSplit parts with a cursor each (workgroup i of the producer writes part
// i % kWideSplit), like the coarse slabs of zen_slab_feed.h and for the same reason: a thousand workgroups
// asking one address wait for each other.
#pragma once

#include "zen_slab.h"
#include "zen_slab_feed.h"

namespace zen {

constexpr int kWideBlock = 1024;                    // threads of a bucket's workgroup
constexpr int kWideCap = 16384;                     // records a bucket sorts in LDS
constexpr int kWideSubs = 16384;                    // narrow key ranges inside a bucket (about one record each)
constexpr int kWideTarget = 15360;                  // records a bucket is sized for
constexpr int kWideMaxBuckets = 256;
constexpr int kWideSplit = kCoarseSplit;            // parts of a bucket's slab
constexpr int kWidePad = kCoarsePad;                // words between two part cursors
constexpr uint32_t kWideCursorWords = kWideMaxBuckets * kWideSplit * kWidePad;

// Buckets for `partitions` partitions of a key space of m keys expected to hold about `expected` records, on
// a chip of `cus` compute units; false if the layout does not suit these sizes.  The result is a SlabGeom
// whose sub_shift refers to kWideSubs narrow ranges.
inline bool wide_geometry(int64_t m, int partitions, int64_t expected, int cus, SlabGeom *out) {
  // a table of 4 MB or more: the map at its head takes at most half, the counters behind it less than 1 MB
  if (m < (1ll << 20) || m > 0x7fffffffll || partitions < 1 || partitions > kWideMaxBuckets || m % partitions != 0 ||
      expected < 1)
    return false;
  int64_t most = cus < kWideMaxBuckets ? cus : kWideMaxBuckets;
  // half the chip where that holds the records: a bucket's workgroup wants a compute unit to itself, and the
  // encode's and the merge's workgroups of one step then find room side by side instead of one after the other
  if (most >= 2 * partitions && expected <= most / 2 * (int64_t)kWideTarget) most /= 2;
  int64_t bpp = most / partitions;
  const int64_t npp = m / partitions;
  if (bpp > npp / (4 * (int64_t)kWideSubs)) bpp = npp / (4 * (int64_t)kWideSubs);  // buckets wider than their sub-ranges
  if (bpp < 1) return false;
  const int64_t nb = bpp * partitions;
  if (expected / nb > (int64_t)kWideTarget) return false;
  SlabGeom g;
  g.m = (uint32_t)m;
  g.npp = (uint32_t)npp;
  g.bpp = (uint32_t)bpp;
  g.bpp_mult = (uint32_t)(((uint64_t)bpp << 32) / (uint64_t)npp);
  g.nbuckets = (uint32_t)nb;
  const uint64_t width = ((1ull << 32) + g.bpp_mult - 1) / g.bpp_mult + 1;  // keys per bucket, at most
  g.sub_shift = 0;
  while ((width >> g.sub_shift) >= (uint64_t)kWideSubs) ++g.sub_shift;
  g.inv_m = slab_inverse_below(g.m);
  g.inv_npp = slab_inverse_below(g.npp);
  *out = g;
  return true;
}

// Entries one part of a bucket's slab holds when list_cap entries at most are spread over the buckets like
// hash values.
inline uint32_t wide_part_cap(const SlabGeom &geo, int64_t list_cap) {
  const int64_t share = ceil_div(list_cap, (int64_t)geo.nbuckets * kWideSplit);
  return (uint32_t)((share + share / 4 + 1024 + 63) / 64 * 64);
}

// Counters of the narrow ranges: 16 bits each, two to a word.  Thread t of the workgroup owns ranges
// 16 t .. 16 t + 15 when the counts become running sums; range s is kept at place (s % 16) * 1024 + s / 16, so
// that the lanes of a wave then walk through consecutive halfwords (and the atomics of the counting steps, on
// ranges that a hash picks, spread over the banks whatever the layout).
struct alignas(16) WideCounters {
  uint32_t word[kWideSubs / 2];
  static_assert(kWideSubs == 16 * kWideBlock, "sixteen ranges per thread");
  __device__ static inline uint32_t place(uint32_t sub) { return ((sub & 15u) << 10) | (sub >> 4); }
  __device__ inline const uint16_t *half() const { return reinterpret_cast<const uint16_t *>(word); }
  __device__ inline void clear() {
    for (int i = threadIdx.x; i < kWideSubs / 2; i += kWideBlock) word[i] = 0;
  }
  __device__ inline void count(uint32_t sub) {
    const uint32_t p = place(sub);
    atomicAdd(&word[p >> 1], 1u << (16 * (p & 1u)));
  }
  // takes the next place of range `sub` (after starts() the counters are running cursors)
  __device__ inline uint32_t take(uint32_t sub) {
    const uint32_t p = place(sub), sh = 16 * (p & 1u);
    return (atomicAdd(&word[p >> 1], 1u << sh) >> sh) & 0xffffu;
  }
  // once every record has taken its place the counter of range s holds where the range ends
  __device__ inline uint32_t end_of(uint32_t sub) const { return half()[place(sub)]; }
  __device__ inline uint32_t start_of(uint32_t sub) const { return sub ? half()[place(sub - 1u)] : 0u; }
  // Counts -> exclusive starts, by the whole workgroup; returns the number of records counted and sets *big
  // (a word of LDS, zero before) if any range holds more than `limit` of them; the caller may read *big once
  // it has synchronised.  smem: kWideBlock / 64 + 1 words.
  __device__ inline uint32_t starts(uint32_t *smem, uint32_t limit, uint32_t *big) {
    uint16_t *h = reinterpret_cast<uint16_t *>(word);
    uint32_t c[16];
    uint32_t sum = 0, over = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      c[e] = h[e * kWideBlock + threadIdx.x];
      sum += c[e];
      over |= c[e] > limit;
    }
    uint32_t total;
    if (over) *big = 1u;
    uint32_t run = block_exclusive_scan<uint32_t, kWideBlock>(sum, smem, &total);
    if (total <= 0xffffu) {  // more than the counters hold: the caller gives up anyway
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        h[e * kWideBlock + threadIdx.x] = (uint16_t)run;
        run += c[e];
      }
    }
    return total;
  }
};

// A barrier between the `members` workgroups that share the counter `word` (zero before the first of them
// arrives; every workgroup of the group calls this the same number of times, `round` = 1, 2, ... says which
// call this is).  What the threads of this workgroup have written with stores of agent scope (store_agent
// below) can be read by the other workgroups with load_agent afterwards.  The wait is bounded: a workgroup
// that gives up says so in *status and goes on.  All workgroups of the group must be resident at the same
// time (the callers launch no more workgroups than the chip has compute units and keep other launches of
// theirs from starting in between).
__device__ inline void group_barrier(uint32_t *word, uint32_t members, uint32_t round, int32_t *status) {
  wait_global_acks();  // this wave's stores and atomics have been carried out
  __syncthreads();
  if (threadIdx.x == 0) {
    atomicAdd(word, 1u);
    const uint32_t want = members * round;
    uint32_t spins = 0;
    while (load_fresh(word) < want) {
      if (++spins > kSpinLimit) {
        atomicOr(status, ZEN_STAT_INTERNAL);
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
  }
  __syncthreads();
}

__device__ inline void store_agent(uint32_t *p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline uint32_t load_agent(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}


// ------------------------------------------------------- received entries -> wide buckets (merge side)
//
// A record in a bucket's slab is one 64-bit word: the index's offset from the bucket's first index (below
// 2^23) in bits 0-22, the arrival number (below 2^25) in bits 23-47 and, for bf16, the value in bits 48-63;
// fp32 values travel in a word plane of their own.  One store per record, and a run of eight fills a line.
constexpr uint32_t kWmOffBits = 23, kWmArrBits = 25;
constexpr int kWmPad = 8;  // words between two part cursors
struct WideSlabs {
  uint32_t *cursor;    // [nbuckets * kWideSplit * kWmPad], zero before the scatter; the bucket's workgroup puts them back
  uint2 *rec;          // [nbuckets * kWideSplit * part_cap]
  uint32_t *val32;     // fp32 values (unused for bf16)
  uint32_t part_cap;
};
__device__ inline uint2 wm_pack(uint32_t off, uint32_t arr, uint32_t val16) {
  return make_uint2(off | (arr << kWmOffBits), (arr >> (32 - kWmOffBits)) | (val16 << 16));
}
__device__ inline uint32_t wm_off(uint2 r) { return r.x & ((1u << kWmOffBits) - 1u); }
__device__ inline uint32_t wm_arr(uint2 r) { return (r.x >> kWmOffBits) | ((r.y & 0xffffu) << (32 - kWmOffBits)); }

// What a workgroup of BLOCK threads needs in LDS to scatter a batch of BLOCK * ITEMS list entries.
template <int BLOCK, int ITEMS>
struct WideScatterShared {
  uint32_t cnt[kWideMaxBuckets], pref[kWideMaxBuckets + 1], gbase[kWideMaxBuckets];
  uint32_t lo[kWideMaxBuckets];  // the buckets' first indices (a 64-bit division each)
  uint32_t scan[BLOCK / 64 + 1];
  uint32_t idx[BLOCK * ITEMS];
  uint16_t from[BLOCK * ITEMS];  // place inside the batch (the arrival number, and where the value is)
  uint8_t dst[BLOCK * ITEMS];
  static_assert(kWideMaxBuckets <= 256 && BLOCK * ITEMS <= 65536, "a destination in a byte, a place in a halfword");
};

// The list of received entries the scatter works on.
struct WideList {
  SlabGeom geo;        // buckets over the index range [0, dense_n)
  const void *idx;     // int32 or int64
  const void *val;     // values in the type S of the caller's template
  uint32_t r, dense_n;
  int idx64;
  WideSlabs out;
  int32_t *status;     // BAD_INDEX, RETRY
};

// Called by the whole workgroup once before its first batch: the buckets' first indices.
template <int BLOCK, int ITEMS>
__device__ inline void wide_scatter_prepare(const WideList &a, WideScatterShared<BLOCK, ITEMS> &sh) {
  for (uint32_t b = threadIdx.x; b < (uint32_t)kWideMaxBuckets; b += BLOCK)
    sh.lo[b] = b < a.geo.nbuckets ? a.geo.first_key(b) : 0u;
  __syncthreads();
}

// Batch number `batch` of the list (BLOCK * ITEMS entries) goes to the buckets' slabs: the workgroup orders
// the entries by bucket in LDS, reserves one run per bucket behind the cursor of part `part` and writes the
// runs with consecutive lanes on consecutive records.  Entries whose index lies outside [0, dense_n) are
// skipped and flagged.  Ends with a barrier.
template <typename S, int BLOCK, int ITEMS>
__device__ inline void wide_scatter_batch(const WideList &a, uint32_t batch, uint32_t part,
                                          WideScatterShared<BLOCK, ITEMS> &sh) {
  constexpr uint32_t kNone = 0xffffffffu;
  const uint32_t first = batch * (uint32_t)(BLOCK * ITEMS);
  const uint32_t nb = a.geo.nbuckets;
  const S *val = static_cast<const S *>(a.val);
  for (uint32_t b = threadIdx.x; b < (uint32_t)kWideMaxBuckets; b += BLOCK) sh.cnt[b] = 0;
  __syncthreads();
  uint32_t k[ITEMS], d[ITEMS], rank[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t e = first + threadIdx.x + i * BLOCK;
    d[i] = kNone;
    k[i] = rank[i] = 0;
    if (e < a.r) {
      const int64_t v = a.idx64 ? static_cast<const int64_t *>(a.idx)[e] : (int64_t)static_cast<const int32_t *>(a.idx)[e];
      if (v < 0 || v >= (int64_t)a.dense_n) {
        atomicOr(a.status, ZEN_STAT_BAD_INDEX);  // skipped, like everything behind the good ones in the general path
      } else {
        k[i] = (uint32_t)v;
        d[i] = a.geo.bucket_of(k[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < ITEMS; ++i)
    if (d[i] != kNone) rank[i] = atomicAdd(&sh.cnt[d[i]], 1u);
  __syncthreads();
  uint32_t total = 0;
  for (uint32_t b0 = 0; b0 < (uint32_t)kWideMaxBuckets; b0 += BLOCK) {  // one turn unless BLOCK < 256
    const uint32_t b = b0 + threadIdx.x;
    const uint32_t c = b < nb ? sh.cnt[b] : 0u;
    uint32_t turn;
    const uint32_t before = total + block_exclusive_scan<uint32_t, BLOCK>(c, sh.scan, &turn);
    if (b < nb) {
      sh.pref[b] = before;
      sh.gbase[b] = c ? atomicAdd(&a.out.cursor[(b * kWideSplit + part) * kWmPad], c) : 0u;
    }
    total += turn;
  }
  if (threadIdx.x == 0) sh.pref[nb] = total;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (d[i] != kNone) {
      const uint32_t p = sh.pref[d[i]] + rank[i];
      sh.idx[p] = k[i];
      sh.from[p] = (uint16_t)(threadIdx.x + i * BLOCK);
      sh.dst[p] = (uint8_t)d[i];
    }
  }
  __syncthreads();
#pragma unroll 2
  for (uint32_t p = threadIdx.x; p < total; p += BLOCK) {
    const uint32_t g = sh.dst[p];
    const uint32_t at = sh.gbase[g] + (p - sh.pref[g]);
    if (at < a.out.part_cap) {
      const size_t o = (size_t)(g * kWideSplit + part) * a.out.part_cap + at;
      const uint32_t e = first + sh.from[p];
      const S v = val[e];  // the batch's arrival numbers are consecutive: these loads hit what it has just read
      a.out.rec[o] = wm_pack(sh.idx[p] - sh.lo[g], e, sizeof(S) == 2 ? (uint32_t)v : 0u);
      if (sizeof(S) == 4) a.out.val32[o] = (uint32_t)v;
    } else {
      atomicOr(a.status, ZEN_STAT_RETRY);  // a slab is full: another path answers
    }
  }
  __syncthreads();
}

// Launches that need all their workgroups resident at once must not be dispatched side by side (each could
// end up holding a part of the chip and waiting for the rest): the host keeps them in line with an event per
// device.  wide_line_enter makes `stream` wait for the last such launch, wide_line_leave records the new one.
// Both do nothing while the stream is being captured into a graph.
int wide_line_enter(hipStream_t stream);
int wide_line_leave(hipStream_t stream);
int wide_device_cus();

// zen_wide_merge.hip
bool wide_merge_fits(int64_t r, int64_t dense_n, int cus, SlabGeom *geo);
size_t wide_merge_bytes(int64_t r, int64_t dense_n, int cus);
bool wide_merge_list(const void *idx, int idx64_in, const void *val, int64_t r, int64_t dense_n, uint32_t *cursor,
                     void *rest, int cus, int32_t *status, WideList *list);
int wide_merge(const WideList &list, int dtype, bool scattered, void *out_idx, int idx64_out, float *out_val,
               int64_t capacity, int64_t *out_count, unsigned long long *scan, hipStream_t s);

}  // namespace zen
