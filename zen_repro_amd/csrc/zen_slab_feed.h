// Moving an unordered list of keyed entries into bucket slabs (zen_slab.h), shared by the encode and the
// merge side.
//
// A direct scatter into a thousand slabs would write runs of three or four records, and memory serves such
// stores one request at a time.  So the list goes to at most 64 coarse slabs first (a coarse slab = `per`
// neighbouring buckets; k_coarse_scatter, or the producer of the entries itself in the same manner: the select
// kernel of the encode side does) and each coarse slab to its buckets afterwards (k_fine_scatter): a
// workgroup orders its 4096 entries by destination in LDS, reserves one run per destination with one atomic
// each and writes runs of dozens to hundreds of entries.  The order inside a slab is whatever the atomics make
// it; the per-bucket sorts that follow do not depend on it.
//
// Atomics on one address are carried out one after the other (about 11 ns each), and a thousand workgroups
// asking the same 64 cursors at once would wait 10 us for that alone: a coarse slab is therefore kept in
// kCoarseSplit parts with a cursor each (workgroup i writes part i % kCoarseSplit), every coarse cursor has a
// 128-byte line to itself, and the bucket cursors sit kCursorPad words apart.  Eight parts: workgroups are
// dealt to the chip's eight dies in turn, so the lines at the growing end of a part are mostly filled by
// workgroups of one die, inside its L2 (measured: the select kernel writes 31 MB instead of 33 for 23 MB of
// candidates and is 2 us shorter).
//
// An entry travels as W 32-bit words, the last of which is kept in memory as the narrower type Src::Last (a
// bf16 value takes two bytes on its way, not four).  What they are comes from two small functor types:
//   Src:   bool load(uint32_t e, uint32_t (&w)[W], uint32_t *bucket)   words and bucket of list entry e;
//                                                                      false: the entry is dropped
//          kStaged, uint32_t late(const uint32_t (&w)[W], int q)       only the first kStaged words go through
//                                                                      LDS in the first step; word q >= kStaged
//                                                                      is asked for again when the entry is
//                                                                      written (from the words before it), so
//                                                                      that more workgroups fit a compute unit
//   Sink:  bool keep(const uint32_t (&w)[W])                           false: the entry is dropped after all
//          uint32_t bucket(const uint32_t (&w)[W])                     the bucket again, from the words
//          void store(size_t at, const uint32_t (&w)[W])               the record at slab place `at`
#pragma once

#include "zen_slab.h"

namespace zen {

constexpr int kFeedItems = 8;
constexpr int kFeedBatch = kSlabBlock * kFeedItems;  // list entries per workgroup
constexpr int kCoarseMax = 64;
constexpr int kCoarsePer = kSlabMaxBuckets / kCoarseMax;  // buckets per coarse slab, at most
constexpr int kCoarsePad = 32;   // words between two coarse cursors
constexpr int kCoarseSplit = 8;  // parts of a coarse slab
constexpr int kCursorPad = 8;    // words between two bucket cursors

struct CoarseGeom {
  uint32_t groups;  // coarse slabs (<= kCoarseMax)
  uint32_t per;     // buckets per coarse slab (<= kCoarsePer)
  uint32_t cap;     // entries one part of a coarse slab holds
  float inv_per;    // (1 / per)(1 - 2^-20), rounded down
};

// list_cap entries at most, spread over the buckets like hash values: a coarse slab receives its share give
// or take a few hundred, and its parts equal shares of that.
inline CoarseGeom coarse_geometry(const SlabGeom &geo, int64_t list_cap) {
  CoarseGeom c;
  c.per = (geo.nbuckets + kCoarseMax - 1) / kCoarseMax;
  c.groups = (geo.nbuckets + c.per - 1) / c.per;
  c.inv_per = slab_inverse_below(c.per);
  const int64_t share = ceil_div(list_cap * c.per, (int64_t)geo.nbuckets * kCoarseSplit);
  c.cap = (uint32_t)(share + share / 8 + 4096);
  return c;
}

inline uint32_t feed_batches(int64_t entries) { return (uint32_t)ceil_div(entries > 0 ? entries : 1, kFeedBatch); }

// Workspace of the two steps.
struct FeedBuffers {
  uint32_t *coarse_cursor;  // [feed_coarse_cursor_words()], zero before the first step (the consumer of the
                            // bucket slabs puts it back to zero)
  uint32_t *coarse_words;   // [W][groups * kCoarseSplit * cap]; the last plane holds Src::Last, not words
  uint32_t *cursor;         // [nbuckets * kCursorPad], zero before the second step; ends as the slab fill counts
                            // (the consumer of a slab puts its count back to zero)
  uint32_t *bucket_lo;      // [nbuckets] smallest key of every bucket (written by the second step)
};
constexpr uint32_t kCoarseCursorWords = kCoarseMax * kCoarseSplit * kCoarsePad;
inline size_t feed_coarse_cursor_words() { return kCoarseCursorWords; }
inline size_t feed_coarse_words(const CoarseGeom &cg, int words) {
  return (size_t)words * cg.groups * kCoarseSplit * cg.cap;
}

// Number of list entries: *list_count if given, never more than list_cap.
__device__ inline uint32_t feed_count(const uint32_t *list_count, uint32_t list_cap) {
  if (!list_count) return list_cap;
  const uint32_t c = *list_count;
  return c < list_cap ? c : list_cap;
}

// Orders the (up to kFeedBatch) live entries of a workgroup by destination d < NDST <= 64 and reserves, per
// destination, a run behind `cursor_of(d)`.  On return s_pref[d] is where destination d starts in the ordered
// batch (s_pref[NDST] = live entries) and s_gbase[d] where its run starts in the destination.
template <int NDST, typename CursorOf>
__device__ inline void feed_runs(const uint32_t (&dst)[kFeedItems], uint32_t (&rank)[kFeedItems], uint32_t *s_cnt,
                                 uint32_t *s_pref, uint32_t *s_gbase, CursorOf cursor_of) {
  static_assert(NDST <= 64, "one wave scans the destinations");
  if (threadIdx.x < NDST) s_cnt[threadIdx.x] = 0;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) rank[i] = dst[i] != 0xffu ? atomicAdd(&s_cnt[dst[i]], 1u) : 0u;
  __syncthreads();
  if (threadIdx.x < 64) {
    const uint32_t n = threadIdx.x < NDST ? s_cnt[threadIdx.x] : 0u;
    const uint32_t incl = wave_inclusive_scan(n);
    if (threadIdx.x < NDST) {
      s_pref[threadIdx.x] = incl - n;
      s_gbase[threadIdx.x] = n ? atomicAdd(cursor_of(threadIdx.x), n) : 0u;
    }
    if (threadIdx.x == NDST - 1) s_pref[NDST] = incl;
  }
  __syncthreads();
}

template <int W, typename Src>
__global__ __launch_bounds__(kSlabBlock) void k_coarse_scatter(SlabGeom geo, CoarseGeom cg, Src src,
                                                               const uint32_t *__restrict__ list_count,
                                                               uint32_t list_cap, uint32_t *__restrict__ coarse_cursor,
                                                               uint32_t *__restrict__ coarse_words, int32_t *status) {
  constexpr int WS = Src::kStaged;
  static_assert(WS >= 1 && WS <= W, "staged words");
  __shared__ uint32_t s_cnt[kCoarseMax], s_pref[kCoarseMax + 1], s_gbase[kCoarseMax];
  __shared__ uint32_t s_word[WS][kFeedBatch];
  __shared__ uint8_t s_dst[kFeedBatch];
  if (list_count && *list_count > list_cap && blockIdx.x == 0 && threadIdx.x == 0)
    atomicOr(status, ZEN_STAT_RETRY);  // the list lost entries
  const uint32_t count = feed_count(list_count, list_cap);
  const uint32_t batch = blockIdx.x * (uint32_t)kFeedBatch;
  if (batch >= count) return;
  const uint32_t part = blockIdx.x % kCoarseSplit;
  uint32_t w[kFeedItems][W], dst[kFeedItems], rank[kFeedItems];
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    const uint32_t e = batch + threadIdx.x + i * kSlabBlock;
    dst[i] = 0xffu;
    uint32_t bucket = 0;
    if (e < count && src.load(e, w[i], &bucket)) {
      uint32_t rem;
      dst[i] = SlabGeom::div_small(bucket, cg.per, cg.inv_per, &rem);
    }
  }
  feed_runs<kCoarseMax>(dst, rank, s_cnt, s_pref, s_gbase,
                        [&](uint32_t d) { return &coarse_cursor[(d * kCoarseSplit + part) * kCoarsePad]; });
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    if (dst[i] != 0xffu) {
      const uint32_t p = s_pref[dst[i]] + rank[i];
#pragma unroll
      for (int q = 0; q < WS; ++q) s_word[q][p] = w[i][q];
      s_dst[p] = (uint8_t)dst[i];
    }
  }
  __syncthreads();
  const uint32_t total = s_pref[kCoarseMax];
  const size_t plane = (size_t)cg.groups * kCoarseSplit * cg.cap;  // words of one word plane
  for (uint32_t p = threadIdx.x; p < total; p += kSlabBlock) {
    const uint32_t d = s_dst[p];
    const uint32_t at = s_gbase[d] + (p - s_pref[d]);
    if (at < cg.cap) {
      const size_t o = (size_t)(d * kCoarseSplit + part) * cg.cap + at;
      uint32_t rec[W];
#pragma unroll
      for (int q = 0; q < WS; ++q) rec[q] = s_word[q][p];
#pragma unroll
      for (int q = WS; q < W; ++q) rec[q] = src.late(rec, q);
#pragma unroll
      for (int q = 0; q < W - 1; ++q) coarse_words[q * plane + o] = rec[q];
      reinterpret_cast<typename Src::Last *>(coarse_words + (size_t)(W - 1) * plane)[o] = (typename Src::Last)rec[W - 1];
    } else {
      atomicOr(status, ZEN_STAT_RETRY);  // a coarse slab is full: the general path answers
    }
  }
}

// Grid: (batches per part, parts of all coarse slabs).  Also writes bucket_lo for the coarse slab's buckets.
template <int W, typename Last, typename Sink>
__global__ __launch_bounds__(kSlabBlock) void k_fine_scatter(SlabGeom geo, CoarseGeom cg, Sink sink,
                                                             const uint32_t *__restrict__ coarse_cursor,
                                                             const uint32_t *__restrict__ coarse_words,
                                                             uint32_t *__restrict__ cursor,
                                                             uint32_t *__restrict__ bucket_lo, uint32_t *clear,
                                                             uint32_t clear_words, int32_t *status) {
  __shared__ uint32_t s_cnt[kCoarsePer], s_pref[kCoarsePer + 1], s_gbase[kCoarsePer];
  // counters of the kernel that filled the coarse slabs, which the caller wants back at zero: a slice per workgroup
  for (uint32_t i = (blockIdx.y * gridDim.x + blockIdx.x) * kSlabBlock + threadIdx.x; i < clear_words;
       i += gridDim.x * gridDim.y * kSlabBlock)
    clear[i] = 0;
  __shared__ uint32_t s_word[W - 1][kFeedBatch];
  __shared__ Last s_last[kFeedBatch];  // the last word in its own type here too: LDS decides how many workgroups share a compute unit
  __shared__ uint8_t s_dst[kFeedBatch];
  const uint32_t c = blockIdx.y / kCoarseSplit;
  const uint32_t first_bucket = c * cg.per;
  if (blockIdx.x == 0 && blockIdx.y % kCoarseSplit == 0 && threadIdx.x < cg.per &&
      first_bucket + threadIdx.x < geo.nbuckets)
    bucket_lo[first_bucket + threadIdx.x] = geo.first_key(first_bucket + threadIdx.x);  // a 64-bit division: once per bucket
  uint32_t count = coarse_cursor[blockIdx.y * kCoarsePad];
  if (count > cg.cap) count = cg.cap;  // the first step flagged the overflow
  const uint32_t batch = blockIdx.x * (uint32_t)kFeedBatch;
  if (batch >= count) return;
  const size_t plane = (size_t)cg.groups * kCoarseSplit * cg.cap;
  const uint32_t *from = coarse_words + (size_t)blockIdx.y * cg.cap;
  const Last *from_last = reinterpret_cast<const Last *>(coarse_words + (size_t)(W - 1) * plane) + (size_t)blockIdx.y * cg.cap;
  uint32_t w[kFeedItems][W], dst[kFeedItems], rank[kFeedItems];
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    const uint32_t e = batch + threadIdx.x + i * kSlabBlock;
    dst[i] = 0xffu;
    if (e < count) {
#pragma unroll
      for (int q = 0; q < W - 1; ++q) w[i][q] = from[q * plane + e];
      w[i][W - 1] = (uint32_t)from_last[e];
      dst[i] = 0;
    }
  }
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i)
    if (dst[i] != 0xffu) dst[i] = sink.keep(w[i]) ? sink.bucket(w[i]) - first_bucket : 0xffu;
  feed_runs<kCoarsePer>(dst, rank, s_cnt, s_pref, s_gbase,
                        [&](uint32_t d) { return &cursor[(first_bucket + d) * kCursorPad]; });
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    if (dst[i] != 0xffu) {
      const uint32_t p = s_pref[dst[i]] + rank[i];
#pragma unroll
      for (int q = 0; q < W - 1; ++q) s_word[q][p] = w[i][q];
      s_last[p] = (Last)w[i][W - 1];
      s_dst[p] = (uint8_t)dst[i];
    }
  }
  __syncthreads();
  const uint32_t total = s_pref[kCoarsePer];
  for (uint32_t p = threadIdx.x; p < total; p += kSlabBlock) {
    const uint32_t d = s_dst[p];
    const uint32_t at = s_gbase[d] + (p - s_pref[d]);
    if (at < (uint32_t)kSlabCap) {
      uint32_t rec[W];
#pragma unroll
      for (int q = 0; q < W - 1; ++q) rec[q] = s_word[q][p];
      rec[W - 1] = (uint32_t)s_last[p];
      sink.store((size_t)(first_bucket + d) * kSlabCap + at, rec);
    } else {
      atomicOr(status, ZEN_STAT_RETRY);  // a slab is full: the general path answers
    }
  }
}

// Launches the second step alone (for a producer that fills the coarse slabs itself), and the two steps.  The
// cursors in `fb` must be zero before the coarse slabs are filled.
template <int W, typename Last, typename Sink>
int feed_fine(const SlabGeom &geo, const CoarseGeom &cg, const Sink &sink, const FeedBuffers &fb, int32_t *status,
              hipStream_t s, uint32_t *clear = nullptr, uint32_t clear_words = 0) {
  k_fine_scatter<W, Last, Sink><<<dim3(feed_batches(cg.cap), cg.groups * kCoarseSplit), dim3(kSlabBlock), 0, s>>>(
      geo, cg, sink, fb.coarse_cursor, fb.coarse_words, fb.cursor, fb.bucket_lo, clear, clear_words, status);
  ZEN_LAUNCH_CHECK("k_fine_scatter");
  return ZEN_OK;
}

template <int W, typename Src, typename Sink>
int feed_slabs(const SlabGeom &geo, const CoarseGeom &cg, const Src &src, const Sink &sink,
               const uint32_t *list_count, int64_t list_cap, const FeedBuffers &fb, int32_t *status, hipStream_t s) {
  k_coarse_scatter<W, Src><<<dim3(feed_batches(list_cap)), dim3(kSlabBlock), 0, s>>>(
      geo, cg, src, list_count, (uint32_t)list_cap, fb.coarse_cursor, fb.coarse_words, status);
  ZEN_LAUNCH_CHECK("k_coarse_scatter");
  return feed_fine<W, typename Src::Last, Sink>(geo, cg, sink, fb, status, s);
}

}  // namespace zen
