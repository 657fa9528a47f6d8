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
  if (m < (1ll << 22) || m > 0x7fffffffll || partitions < 1 || partitions > kWideMaxBuckets || m % partitions != 0 ||
      expected < 1)
    return false;
  int64_t most = cus < kWideMaxBuckets ? cus : kWideMaxBuckets;
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

// The parts of a bucket's slab as one sequence of records: where record j of the sequence sits.
struct WideParts {
  uint32_t cum[kWideSplit + 1];  // records in the parts before part q
  uint32_t first;                // number of the bucket's first part
  uint32_t cap;                  // entries a part holds
  __device__ inline uint32_t total() const { return cum[kWideSplit]; }
  __device__ inline size_t place(uint32_t j) const {
    uint32_t q = 0, base = 0;
#pragma unroll
    for (int i = 1; i < kWideSplit; ++i) {
      const bool past = j >= cum[i];
      q += past;
      base = past ? cum[i] : base;
    }
    return (size_t)(first + q) * cap + (j - base);
  }
};

// Reads the part counts of bucket b (clamped to the parts' capacity: the producer flagged the overflow).
__device__ inline WideParts wide_parts(const uint32_t *cursor, uint32_t b, uint32_t cap) {
  WideParts p;
  p.first = b * kWideSplit;
  p.cap = cap;
  uint32_t c[kWideSplit];
#pragma unroll
  for (int q = 0; q < kWideSplit; ++q) c[q] = cursor[(b * kWideSplit + q) * kWidePad];
  p.cum[0] = 0;
#pragma unroll
  for (int q = 0; q < kWideSplit; ++q) p.cum[q + 1] = p.cum[q] + (c[q] < cap ? c[q] : cap);
  return p;
}

// Counters of the narrow ranges: 16 bits each, two to a word, with a zero in front of the first (the end of
// "range -1"), so that range s spans [cnt[s - 1], cnt[s]) once the counters have become running ends.
struct alignas(16) WideCounters {
  uint32_t pad[4];                 // cnt16[-8 .. -1]: stays zero
  uint32_t word[kWideSubs / 2];    // cnt16[0 .. kWideSubs)
  __device__ inline uint16_t *cnt16() { return reinterpret_cast<uint16_t *>(word); }
  __device__ inline void clear() {
    uint32_t *all = reinterpret_cast<uint32_t *>(this);
    for (int i = threadIdx.x; i < kWideSubs / 2 + 4; i += kWideBlock) all[i] = 0;
  }
  __device__ inline void count(uint32_t sub) { atomicAdd(&word[sub >> 1], 1u << (16 * (sub & 1u))); }
  // takes the next place of range `sub` (after starts() the counters are running cursors)
  __device__ inline uint32_t take(uint32_t sub) {
    const uint32_t sh = 16 * (sub & 1u);
    return (atomicAdd(&word[sub >> 1], 1u << sh) >> sh) & 0xffffu;
  }
  // Counts -> exclusive starts, by the whole workgroup (thread t owns ranges 16 t .. 16 t + 15); returns the
  // number of records counted.  smem: kWideBlock / 64 + 1 words.
  __device__ inline uint32_t starts(uint32_t *smem) {
    static_assert(kWideSubs == 16 * kWideBlock, "sixteen ranges per thread");
    uint4 *mine = reinterpret_cast<uint4 *>(word) + 2 * threadIdx.x;
    const uint4 a = mine[0], b = mine[1];
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += (w[i] & 0xffffu) + (w[i] >> 16);
    uint32_t total;
    uint32_t run = block_exclusive_scan<uint32_t, kWideBlock>(sum, smem, &total);
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t lo = run;
      run += w[i] & 0xffffu;
      const uint32_t hi = run;
      run += w[i] >> 16;
      o[i] = (lo & 0xffffu) | (hi << 16);
    }
    if (total <= 0xffffu) {  // more than the counters hold: the caller gives up anyway
      mine[0] = make_uint4(o[0], o[1], o[2], o[3]);
      mine[1] = make_uint4(o[4], o[5], o[6], o[7]);
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

// Launches that need all their workgroups resident at once must not be dispatched side by side (each could
// end up holding a part of the chip and waiting for the rest): the host keeps them in line with an event per
// device.  wide_line_enter makes `stream` wait for the last such launch, wide_line_leave records the new one.
// Both do nothing while the stream is being captured into a graph.
int wide_line_enter(hipStream_t stream);
int wide_line_leave(hipStream_t stream);
int wide_device_cus();

}  // namespace zen
