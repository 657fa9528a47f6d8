// Bucket slabs: the layout both fast paths (encode and merge) are built on.
//
// Keys that spread evenly over a range -- level-1 hash slots on the encode
// side, hashed indices arriving at one destination on the merge side -- are
// cut into `nbuckets` contiguous key ranges of equal width.  Every bucket owns
// a slab of kSlabCap records in the workspace.  The producer kernel appends
// records to the slabs in whatever order they turn up (one cursor per bucket,
// reserved once per staged batch and bucket); afterwards one workgroup per
// bucket sorts its slab inside LDS.  Buckets never straddle a partition
// (nbuckets = partitions * buckets-per-partition), so bucket order is output
// order.  A slab that overflows raises ZEN_STAT_RETRY and the caller falls
// back to the general (radix sort) path.
#pragma once

#include <math.h>

#include "zen_common.h"

namespace zen {

constexpr uint32_t kRemovedBit = 1u << 31;  // in a sorted index word: the entry lost its level-1 slot
constexpr uint32_t kIndexMask = kRemovedBit - 1u;

constexpr int kSlabBlock = 512;                       // threads of a per-bucket workgroup (the sort takes twice as many)
constexpr int kSlabItems = 12;                        // records per thread
constexpr int kSlabCap = kSlabBlock * kSlabItems;     // records per slab (6144)
constexpr int kSlabSubs = 4096;                       // narrow key ranges inside a bucket (about one record each)
constexpr int kSlabMaxBlock = 1024;                   // largest workgroup that ranks a slab
constexpr int kSlabGroupLimit = 1024;                 // bounds the rank loop on piled-up keys
constexpr int kSlabMaxBuckets = 4096;
constexpr int kSlabTarget = 3584;                     // records a bucket is sized for (leaves 40 % to spare)
constexpr int kSlabResident = 512;                    // per-bucket workgroups the chip holds at a time (256 CUs x 2)
constexpr int kSlabMoveCap = 1024;                    // entries that may move into one bucket from elsewhere
constexpr int kSlabSerialCap = 4096;                  // overflow entries per partition the fast path carries

struct SlabGeom {
  uint32_t m;         // keys are < m
  uint32_t npp;       // keys per partition (m / partitions)
  uint32_t bpp;       // buckets per partition
  uint32_t bpp_mult;  // floor(bpp * 2^32 / npp)
  uint32_t nbuckets;  // partitions * bpp
  int sub_shift;      // key offset inside a bucket >> sub_shift = narrow range (fewer than kSlabSubs of them)
  float inv_m;        // (1 / m)(1 - 2^-20), rounded down
  float inv_npp;      // the same for npp

  // x / d for x < 2^32 and quotients below 2^11, without the long integer division sequence.  `inv` is
  // (1 / d)(1 - 2^-20): the two roundings of the float estimate (each at most 2^-24, relative) cannot lift it
  // above x / d, and it falls short by less than 2^11 * 2^-19: it is the quotient or one less.
  __device__ static inline uint32_t div_small(uint32_t x, uint32_t d, float inv, uint32_t *rem) {
    uint32_t q = (uint32_t)((float)x * inv);
    uint32_t r = x - q * d;
    if (r >= d) {
      r -= d;
      ++q;
    }
    *rem = r;
    return q;
  }
  __device__ inline uint32_t mod_m(uint32_t h) const {  // h % m
    uint32_t r;
    div_small(h, m, inv_m, &r);
    return r;
  }
  __device__ inline uint32_t bucket_of(uint32_t key) const {
    uint32_t local;
    const uint32_t part = div_small(key, npp, inv_npp, &local);
    return part * bpp + __umulhi(local, bpp_mult);
  }
  __device__ inline uint32_t first_key(uint32_t b) const {  // smallest key of bucket b
    const uint32_t part = b / bpp, sb = b - part * bpp;
    return part * npp + (uint32_t)((((uint64_t)sb << 32) + bpp_mult - 1) / bpp_mult);
  }
};

// Host side: geometry for `partitions` partitions of a key space of m keys (m a
// multiple of partitions) expected to hold about `expected` records.  Returns
// false if the slab layout does not suit these sizes.
inline float slab_inverse_below(uint32_t d) {
  const double want = (1.0 / (double)d) * (1.0 - 1.0 / 1048576.0);
  float f = (float)want;
  while ((double)f > want) f = nextafterf(f, 0.0f);
  return f;
}

inline bool slab_geometry(int64_t m, int partitions, int64_t expected, int target, SlabGeom *out) {
  if (m < (1ll << 22) || m > 0x7fffffffll || partitions < 1 || partitions > kSlabMaxBuckets || m % partitions != 0 ||
      expected < 1)
    return false;
  int64_t bpp = ceil_div(expected, (int64_t)target * partitions);
  if (bpp < 1) bpp = 1;
  if (bpp * partitions > kSlabMaxBuckets) bpp = kSlabMaxBuckets / partitions;
  // The per-bucket kernels run in rounds of kSlabResident workgroups, and a workgroup costs much the same whether
  // its slab is half or three quarters full: a bucket count a little above a whole number of rounds wastes most
  // of the last one.  Fewer, fuller buckets then do better, as long as a slab keeps a quarter to spare.
  {
    const int64_t rounds = ceil_div(bpp * partitions, (int64_t)kSlabResident);
    const int64_t fewer = (rounds - 1) * kSlabResident / partitions;
    if (fewer >= 1 && expected / (fewer * partitions) <= (int64_t)kSlabCap * 3 / 4) bpp = fewer;
  }
  const int64_t nb = bpp * partitions;
  if (expected / nb > (int64_t)kSlabCap * 3 / 4) return false;  // too many records per bucket
  const int64_t npp = m / partitions;
  if (npp / bpp < 4 * kSlabSubs) return false;                  // buckets narrower than their sub-ranges
  SlabGeom g;
  g.m = (uint32_t)m;
  g.npp = (uint32_t)npp;
  g.bpp = (uint32_t)bpp;
  g.bpp_mult = (uint32_t)(((uint64_t)bpp << 32) / (uint64_t)npp);
  g.nbuckets = (uint32_t)nb;
  const uint64_t width = ((1ull << 32) + g.bpp_mult - 1) / g.bpp_mult + 1;  // keys per bucket, at most
  g.sub_shift = 0;
  while ((width >> g.sub_shift) >= (uint64_t)kSlabSubs) ++g.sub_shift;
  g.inv_m = slab_inverse_below(g.m);
  g.inv_npp = slab_inverse_below(g.npp);
  *out = g;
  return true;
}

// Where the counter of narrow range s lives in SlabSortShared::cnt when BLOCK threads rank the slab: a thread
// owns kSlabSubs / BLOCK consecutive ranges during the prefix step, and this keeps the lanes of a wave on
// different LDS banks while they walk through their ranges.  Range kSlabSubs (the end marker) stays at index
// kSlabSubs.
template <int BLOCK>
__device__ inline uint32_t sub_place(uint32_t s) {
  constexpr uint32_t kPer = kSlabSubs / BLOCK;
  return s < (uint32_t)kSlabSubs ? (s % kPer) * BLOCK + s / kPer : s;
}

// Shared memory of the in-LDS sort.  slab_rank does not touch `tie`, and a caller that fills it only after
// slab_rank has returned and has no use for `cnt` from then on lets the two share their memory (OVERLAY):
// LDS decides how many workgroups share a compute unit.
template <bool OVERLAY>
struct SlabSortSharedT;
constexpr int kSlabQueueCap = kSlabCap - kSlabSubs - 1;  // large-group records a workgroup sets aside
constexpr int kSlabInline = 4;                            // groups up to this size are ranked by their own threads
constexpr int kSlabQueueMin = 256;                        // records in larger groups below which nothing is set aside
template <>
struct SlabSortSharedT<false> {
  static constexpr bool kQueue = false;
  uint32_t key[kSlabCap];
  uint32_t tie[kSlabCap];
  uint32_t cnt[kSlabSubs + 1];
  uint32_t scan[kSlabMaxBlock / 64 + 1];
  uint32_t bad;
};
template <>
struct SlabSortSharedT<true> {
  static constexpr bool kQueue = true;
  uint32_t key[kSlabCap];
  union {
    uint32_t tie[kSlabCap];
    struct {
      uint32_t cnt[kSlabSubs + 1];
      uint32_t queue[kSlabQueueCap];  // the rest of the ties' memory: records of large groups (see slab_rank)
    };
  };
  uint32_t scan[kSlabMaxBlock / 64 + 1];
  uint32_t bad;
};

// The same sharing of memory without the queue (the queue's code costs slab_rank registers).
struct SlabSortSharedNoQueue {
  static constexpr bool kQueue = false;
  uint32_t key[kSlabCap];
  union {
    uint32_t tie[kSlabCap];
    uint32_t cnt[kSlabSubs + 1];
  };
  uint32_t scan[kSlabMaxBlock / 64 + 1];
  uint32_t bad;
};

static_assert(kSlabSubs + 1 <= kSlabCap, "the counters fit under the ties");
using SlabSortShared = SlabSortSharedT<false>;

// Number of words in sh.key[b0, b1) that are smaller than w.  The words are fetched four at a time (places past
// the end are pulled back onto the last word and not counted): a loop that fetches one word per turn waits
// for LDS once per word, and that wait is what such a loop spends its time on.
template <typename Shared>
__device__ inline uint32_t slab_count_less(const Shared &sh, uint32_t b0, uint32_t b1, uint32_t w) {
  uint32_t less = 0;
  const uint32_t last = b1 - 1u;
  for (uint32_t u = b0; u < b1; u += 4) {
    const uint32_t a0 = sh.key[u];
    const uint32_t a1 = sh.key[u + 1 < last ? u + 1 : last];
    const uint32_t a2 = sh.key[u + 2 < last ? u + 2 : last];
    const uint32_t a3 = sh.key[u + 3 < last ? u + 3 : last];
    less += (a0 < w) + (u + 1 < b1 && a1 < w) + (u + 2 < b1 && a2 < w) + (u + 3 < b1 && a3 < w);
  }
  return less;
}

// Ranks the live records of a workgroup of BLOCK threads (kSlabCap / BLOCK records each) by (key offset, tie);
// tie < 2^tie_bits, the pair unique, and
// geo.sub_shift + tie_bits <= 32.  off[i] < bucket width.  The records are first grouped by narrow key range
// with one LDS atomic each; a record is then one word, (offset inside the range) << tie_bits | tie, and
// inside its group every record counts the words smaller than its own: the first kSlabInline words of every
// record's group are fetched in one go (all of them in flight together), which settles groups up to that size.
// Where many records share a key (a merge of payloads that overlap) a few lanes of every wave would then walk
// through groups of dozens while the others wait: with a Shared that has a queue, records of groups larger
// than kSlabInline are set aside instead (their places in the queue follow from the same prefix sums as the
// groups' places: the counters carry both, 16 bits each) and handed out again afterwards, one per lane, so
// that the lanes of a wave walk through large groups together.  Returns false (for every thread) if a
// group is too large for that; else rank[i] for live records and *n_out = number of live records.  On return
// sh.key / sh.tie may be overwritten at once (sh.tie is not touched at all), and the low 16 bits of
// sh.cnt[sub_place(s)] hold the sorted place of the first record of narrow range s.
template <int BLOCK, typename Shared>
__device__ inline bool slab_rank(Shared &sh, const SlabGeom &geo, int tie_bits,
                                 const uint32_t (&off)[kSlabCap / BLOCK], const uint32_t (&tie)[kSlabCap / BLOCK],
                                 uint32_t live, uint32_t (&rank)[kSlabCap / BLOCK], uint32_t *n_out) {
  static_assert(BLOCK <= kSlabMaxBlock && kSlabCap % BLOCK == 0 && kSlabSubs % BLOCK == 0, "workgroup size");
  static_assert(kSlabCap < 65536, "two prefixes in one word");
  constexpr int kItems = kSlabCap / BLOCK;
  constexpr int kSubsPer = kSlabSubs / BLOCK;
  for (int d = threadIdx.x; d <= kSlabSubs; d += BLOCK) sh.cnt[d] = 0;
  if (threadIdx.x == 0) sh.bad = 0;
  __syncthreads();
  const uint32_t low_mask = (1u << geo.sub_shift) - 1u;
  uint32_t sub[kItems], at[kItems];
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    sub[i] = at[i] = 0;
    if (live & (1u << i)) {
      sub[i] = off[i] >> geo.sub_shift;
      at[i] = atomicAdd(&sh.cnt[sub_place<BLOCK>(sub[i])], 1u);
    }
  }
  __syncthreads();
  {
    uint32_t c[kSubsPer];
    uint32_t sum = 0, big = 0;  // sum: records in the low half, records of groups larger than kSlabInline in the high half
#pragma unroll
    for (int e = 0; e < kSubsPer; ++e) {
      c[e] = sh.cnt[e * BLOCK + threadIdx.x];
      sum += c[e] + (c[e] > (uint32_t)kSlabInline ? c[e] << 16 : 0u);
      big |= c[e] > (uint32_t)kSlabGroupLimit;
    }
    if (big) sh.bad = 1;
    uint32_t total;
    uint32_t running = block_exclusive_scan<uint32_t, BLOCK>(sum, sh.scan, &total);
#pragma unroll
    for (int e = 0; e < kSubsPer; ++e) {
      sh.cnt[e * BLOCK + threadIdx.x] = running;
      running += c[e] + (c[e] > (uint32_t)kSlabInline ? c[e] << 16 : 0u);
    }
    if (threadIdx.x == BLOCK - 1) sh.cnt[kSlabSubs] = running;  // = total
  }
  __syncthreads();
  if (sh.bad) return false;
  const uint32_t totals = sh.cnt[kSlabSubs];
  // a few large groups are not worth the extra barrier
  const bool set_aside = Shared::kQueue && (totals >> 16) >= (uint32_t)kSlabQueueMin;
  constexpr uint32_t kSetAside = 0x80000000u;
  uint32_t g0[kItems], g1[kItems], word[kItems];
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    g0[i] = g1[i] = word[i] = rank[i] = 0;
    if (live & (1u << i)) {
      const uint32_t here = sh.cnt[sub_place<BLOCK>(sub[i])];
      g0[i] = here & 0xffffu;
      g1[i] = sh.cnt[sub_place<BLOCK>(sub[i] + 1)] & 0xffffu;
      word[i] = ((off[i] & low_mask) << tie_bits) | tie[i];
      sh.key[g0[i] + at[i]] = word[i];
      if constexpr (Shared::kQueue) {
        static_assert(kSlabSubs <= (1 << 12) && kSlabGroupLimit <= (1 << 19), "a queue entry is one word");
        const uint32_t q = (here >> 16) + at[i];
        if (set_aside && g1[i] - g0[i] > (uint32_t)kSlabInline && q < (uint32_t)kSlabQueueCap) {
          sh.queue[q] = sub[i] | (at[i] << 12);  // sub < 2^12, at < group size <= kSlabGroupLimit
          rank[i] = kSetAside | q;
          g1[i] = g0[i];  // nothing left to do for it below
        }
      }
    }
  }
  __syncthreads();
  // the first kRankAhead words of every record's group, those of kBatch records fetched before any is looked
  // at (most groups are no larger); the rest of a group one word per turn, or four where it is large
#ifndef ZEN_RANK_AHEAD
#define ZEN_RANK_AHEAD 2
#endif
  constexpr int kRankAhead = ZEN_RANK_AHEAD;
  constexpr int kBatch = kItems % 3 == 0 ? 3 : kItems;
#pragma unroll
  for (int h = 0; h < kItems; h += kBatch) {
    uint32_t a[kBatch][kRankAhead];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const uint32_t last = g1[h + i] > g0[h + i] ? g1[h + i] - 1u : g0[h + i];
#pragma unroll
      for (int j = 0; j < kRankAhead; ++j) a[i][j] = sh.key[g0[h + i] + j < last ? g0[h + i] + j : last];
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (g1[h + i] > g0[h + i]) {
        uint32_t less = 0;
#pragma unroll
        for (int j = 0; j < kRankAhead; ++j) less += g0[h + i] + j < g1[h + i] && a[i][j] < word[h + i];
        const uint32_t size = g1[h + i] - g0[h + i];
        if (size > (uint32_t)kSlabInline)
          less += slab_count_less(sh, g0[h + i] + kRankAhead, g1[h + i], word[h + i]);
        else
          for (uint32_t u = g0[h + i] + kRankAhead; u < g1[h + i]; ++u) less += sh.key[u] < word[h + i];
        rank[h + i] = g0[h + i] + less;
      }
    }
  }
  if constexpr (Shared::kQueue) {
    if (set_aside) {
      const uint32_t queued = (totals >> 16) < (uint32_t)kSlabQueueCap ? (totals >> 16) : (uint32_t)kSlabQueueCap;
      // the thread that takes a queue entry also overwrites it with the rank
#pragma unroll 1
      for (uint32_t q = threadIdx.x; q < queued; q += BLOCK) {
        const uint32_t e = sh.queue[q];
        const uint32_t b0 = sh.cnt[sub_place<BLOCK>(e & 4095u)] & 0xffffu;
        const uint32_t b1 = sh.cnt[sub_place<BLOCK>((e & 4095u) + 1)] & 0xffffu;
        sh.queue[q] = b0 + slab_count_less(sh, b0, b1, sh.key[b0 + (e >> 12)]);
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < kItems; ++i)
        if (rank[i] & kSetAside) rank[i] = sh.queue[rank[i] & ~kSetAside];
    }
  }
  *n_out = totals & 0xffffu;
  __syncthreads();
  return true;
}

}  // namespace zen
