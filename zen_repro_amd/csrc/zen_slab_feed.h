// Moving an unordered list of keyed entries into bucket slabs (zen_slab.h), shared by the encode and the
// merge side.  Three kernels, no global atomic (a reservation per bucket and batch would be a million
// device-wide atomics, and those on one cache line are carried out one after the other): every workgroup counts
// its batch of the list per bucket (k_feed_count), a scan over the batches turns the counts of a bucket into
// the places where each batch's run starts in the bucket's slab (k_feed_scan), and every workgroup orders its
// batch by bucket in LDS and writes the runs as 16-byte records (k_feed_write).
//
// What an entry is comes from two small functor types:
//   CountSrc:  uint32_t key(uint32_t e)   key of list entry e, or kNoSlot if the entry is dropped (it may
//                                         store the key for the write pass)
//   WriteSrc:  void rec(uint32_t e, uint32_t *key, uint32_t *a, uint32_t *b)   the record of entry e: its key
//                                         (kNoSlot: dropped) and two payload words
#pragma once

#include "zen_slab.h"

namespace zen {

constexpr int kFeedItems = 8;
constexpr int kFeedBatch = kSlabBlock * kFeedItems;  // list entries per workgroup
constexpr int kScanChunks = 32;
constexpr int kScanCols = 8;  // 256 threads: a workgroup this small finds room on a CU other kernels are using
constexpr uint32_t kNoSlot = 0xffffffffu;  // key of an entry that is dropped

// Number of list entries: *list_count if given, never more than list_cap.
__device__ inline uint32_t feed_count(const uint32_t *list_count, uint32_t list_cap) {
  if (!list_count) return list_cap;
  const uint32_t c = *list_count;
  return c < list_cap ? c : list_cap;
}

inline uint32_t feed_row_words(uint32_t nbuckets) { return (nbuckets + 63u) / 64u * 64u; }
inline uint32_t feed_batches(int64_t list_cap) { return (uint32_t)ceil_div(list_cap, kFeedBatch); }
// hist needs feed_batches(list_cap) * feed_row_words(nbuckets) words

template <typename CountSrc>
__global__ __launch_bounds__(kSlabBlock) void k_feed_count(SlabGeom geo, CountSrc src,
                                                           const uint32_t *__restrict__ list_count, uint32_t list_cap,
                                                           uint32_t row_words, uint32_t *__restrict__ hist,
                                                           int32_t *status) {
  __shared__ uint32_t s_cnt[kSlabMaxBuckets];
  if (list_count && *list_count > list_cap && blockIdx.x == 0 && threadIdx.x == 0)
    atomicOr(status, ZEN_STAT_RETRY);  // the list lost entries
  const uint32_t count = feed_count(list_count, list_cap);
  const uint32_t batch = blockIdx.x * (uint32_t)kFeedBatch;
  if (batch >= count) return;
  for (uint32_t b = threadIdx.x; b < row_words; b += kSlabBlock) s_cnt[b] = 0;
  __syncthreads();
  uint32_t key[kFeedItems];
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    const uint32_t e = batch + threadIdx.x + i * kSlabBlock;
    key[i] = e < count ? src.key(e) : kNoSlot;
  }
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i)
    if (key[i] != kNoSlot) atomicAdd(&s_cnt[geo.bucket_of(key[i])], 1u);
  __syncthreads();
  uint32_t *row = hist + (size_t)blockIdx.x * row_words;
  for (uint32_t b = threadIdx.x; b < row_words; b += kSlabBlock) row[b] = s_cnt[b];
}

// Workgroup = kScanCols buckets x kScanChunks ranges of batches.  hist[batch][bucket] becomes the number of the
// bucket's entries in earlier batches; cursor[bucket] = the bucket's total; bucket_lo[bucket] = its first key.
__global__ __launch_bounds__(kScanCols * kScanChunks) void k_feed_scan(SlabGeom geo,
                                                                       const uint32_t *__restrict__ list_count,
                                                                       uint32_t list_cap, uint32_t nbuckets,
                                                                       uint32_t row_words, uint32_t *__restrict__ hist,
                                                                       uint32_t *__restrict__ cursor,
                                                                       uint32_t *__restrict__ bucket_lo,
                                                                       int32_t *status);

// Every kept entry of the batch goes to its bucket's slab as one 16-byte record (key, a, b, 0).  Scattered
// stores cost one memory request each whatever their size (about 80 G requests/s on this part), so the batch
// is first ordered by bucket in LDS: the records of a bucket then leave as one run, a few requests instead of
// one per record.  A run's place in the slab comes from the scan.
template <typename WriteSrc>
__global__ __launch_bounds__(kSlabBlock) void k_feed_write(SlabGeom geo, WriteSrc src,
                                                           const uint32_t *__restrict__ list_count, uint32_t list_cap,
                                                           uint32_t row_words, const uint32_t *__restrict__ hist,
                                                           uint4 *__restrict__ slab_rec) {
  // entries of the batch per bucket; then (where the bucket's run starts in the ordered batch) << 13 | (where it
  // starts in the slab).  One array, so that two workgroups fit into a compute unit's LDS.
  __shared__ uint32_t s_cnt[kSlabMaxBuckets];
  __shared__ uint4 s_rec[kFeedBatch];  // the ordered batch; .w = bucket << 13 | place in the slab
  __shared__ uint32_t s_scan[kSlabBlock / 64 + 1];
  static_assert(kSlabCap <= (1 << 13) && kFeedBatch < (1 << 13) && kSlabMaxBuckets <= (1 << 11), "packed fields");
  const uint32_t count = feed_count(list_count, list_cap);
  const uint32_t batch = blockIdx.x * (uint32_t)kFeedBatch;
  if (batch >= count) return;
  for (uint32_t b = threadIdx.x; b < (uint32_t)kSlabMaxBuckets; b += kSlabBlock) s_cnt[b] = 0;
  // where the runs of this thread's buckets start in the slabs: asked for now, needed after the counting
  constexpr int kPer = kSlabMaxBuckets / kSlabBlock;
  uint32_t base[kPer];
  {
    const uint32_t *row = hist + (size_t)blockIdx.x * row_words;
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      const uint32_t b = threadIdx.x * kPer + e;
      base[e] = b < row_words ? row[b] : 0u;
    }
  }
  __syncthreads();
  uint32_t pa[kFeedItems], pb[kFeedItems], key[kFeedItems], bucket[kFeedItems], rank[kFeedItems];
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    const uint32_t e = batch + threadIdx.x + i * kSlabBlock;
    pa[i] = pb[i] = 0;
    key[i] = kNoSlot;
    if (e < count) src.rec(e, &key[i], &pa[i], &pb[i]);
  }
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    bucket[i] = rank[i] = 0;
    if (key[i] != kNoSlot) {
      bucket[i] = geo.bucket_of(key[i]);
      rank[i] = atomicAdd(&s_cnt[bucket[i]], 1u);
    }
  }
  __syncthreads();
  uint32_t batch_live;
  {
    // thread owns kPer consecutive buckets: one exclusive prefix over the buckets gives every bucket's run a
    // place in the ordered batch
    uint32_t c[kPer];
    uint32_t sum = 0;
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      c[e] = s_cnt[threadIdx.x * kPer + e];
      sum += c[e];
    }
    uint32_t running = block_exclusive_scan<uint32_t, kSlabBlock>(sum, s_scan, &batch_live);
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      // a run that starts past the slab's end (overflow, flagged by the scan) is clipped to the end
      s_cnt[threadIdx.x * kPer + e] = (running << 13) | (base[e] < (uint32_t)kSlabCap ? base[e] : (uint32_t)kSlabCap);
      running += c[e];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kFeedItems; ++i) {
    if (key[i] != kNoSlot) {
      const uint32_t sb = s_cnt[bucket[i]];
      uint32_t pos = (sb & 8191u) + rank[i];
      if (pos > 8191u) pos = 8191u;  // beyond the slab anyway: dropped below, must not spill into the bucket field
      s_rec[(sb >> 13) + rank[i]] = make_uint4(key[i], pa[i], pb[i], (bucket[i] << 13) | pos);
    }
  }
  __syncthreads();
  // consecutive lanes write consecutive records of a run
  for (uint32_t e = threadIdx.x; e < batch_live; e += kSlabBlock) {
    uint4 rec = s_rec[e];
    const uint32_t b = rec.w >> 13, pos = rec.w & 8191u;
    rec.w = 0;
    if (pos < (uint32_t)kSlabCap) slab_rec[(size_t)b * kSlabCap + pos] = rec;
  }
}

// Launches the three kernels.  hist: feed_batches(list_cap) * feed_row_words(nbuckets) words.
template <typename CountSrc, typename WriteSrc>
int feed_slabs(const SlabGeom &geo, const CountSrc &csrc, const WriteSrc &wsrc, const uint32_t *list_count,
               int64_t list_cap, uint32_t *hist, uint32_t *cursor, uint32_t *bucket_lo, uint4 *slab_rec,
               int32_t *status, hipStream_t s) {
  const uint32_t row_words = feed_row_words(geo.nbuckets);
  const unsigned batches = feed_batches(list_cap);
  k_feed_count<CountSrc><<<dim3(batches), dim3(kSlabBlock), 0, s>>>(geo, csrc, list_count, (uint32_t)list_cap, row_words,
                                                                    hist, status);
  ZEN_LAUNCH_CHECK("k_feed_count");
  k_feed_scan<<<dim3(row_words / kScanCols), dim3(kScanCols * kScanChunks), 0, s>>>(
      geo, list_count, (uint32_t)list_cap, geo.nbuckets, row_words, hist, cursor, bucket_lo, status);
  ZEN_LAUNCH_CHECK("k_feed_scan");
  k_feed_write<WriteSrc><<<dim3(batches), dim3(kSlabBlock), 0, s>>>(geo, wsrc, list_count, (uint32_t)list_cap, row_words,
                                                                    hist, slab_rec);
  ZEN_LAUNCH_CHECK("k_feed_write");
  return ZEN_OK;
}

}  // namespace zen
