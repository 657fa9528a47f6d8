// Fused load balance on bucket slabs (the fast path of zen_load_balance).
//
// The reference inserts every selected index into an int32 table as large as
// the gradient and then scans that table partition by partition
// (functions_cuda_kernel.cu:97-167, tensor_load_balance.py:13-51).  Here the
// select kernel leaves its candidates in 64 coarse slabs (a coarse slab = the
// level-1 hash slots of a group of buckets; a bucket is a range of level-1
// slots, zen_slab.h), and five short kernels finish the job:
//   k_fine_scatter  the coarse slabs, filtered by the exact threshold, go to the
//                   bucket slabs, so that every store belongs to a long run;
//   k_slab_sort     one workgroup per bucket: sorts
//                   the bucket by (level-1 slot, index) inside LDS; in a run of
//                   equal slots the first entry (smallest index) is the slot's
//                   level-1 owner, the others lost level 1 and are logged;
//   k_slab_chains   levels 2 and 3 for the losers through a small hash map,
//                   with the reference's rule executed in ascending index order
//                   (a slot belongs to the smallest index that ever probes it;
//                   whoever takes a slot from a larger index continues that
//                   index's probe sequence);
//   k_slab_classify final slot of every logged entry, handed to the bucket that
//                   slot lies in (or to the partition's serial list);
//   k_slab_place    one workgroup per bucket: survivors and moved-in entries
//                   merged by rank, written to the bucket's place in the
//                   partition-major output; split sizes.
#include "zen_balance.h"
#include "zen_hashmap.h"
#include "zen_slab.h"
#include "zen_slab_feed.h"
#include "zen_refine.h"

namespace zen {
namespace {

struct SlabTables {
  uint32_t *cursor;     // [B * kCursorPad] records in the bucket's slab, at [b * kCursorPad]
  uint32_t *bucket_lo;  // [B] smallest level-1 slot of the bucket
  uint32_t *bucket_n;   // [B] selected records, sorted, in the slab
  uint32_t *removed_n;  // [B] of which lost their level-1 slot
  uint32_t *movein_n;   // [B] entries whose final slot lies in the bucket but whose level-1 slot does not own it
  uint32_t *serial_n;   // [P] entries that found no slot
  uint32_t *raw_idx;    // [B * kSlabCap] entries as they arrive: index ...
  void *raw_val;        // ... and value
  int32_t *slab_idx;    // [B * kSlabCap] after the sort: index | kRemovedBit, by ascending level-1 slot (the slot
                        // itself is not kept: hashing the index again is cheaper than a trip to memory)
  void *slab_val;       // [B * kSlabCap] after the sort: value
  uint16_t *sub_index;  // [B * kSlabIndexLen] sorted place of the first record of every kSlabIndexStep-th narrow
                        // key range of the bucket (the last entry: the number of records)
  uint32_t *mv_key, *mv_idx, *mv_val;  // [B * kSlabMoveCap]
  uint32_t *ser_idx;    // [P * kSlabSerialCap]
  uint32_t *log_t, *log_v, *log_cell;  // [log_cap]
  uint32_t *out_start;  // [B + 1] where every bucket starts in the output
  uint32_t *done;       // [1] workgroups of k_slab_classify that have finished
  uint32_t *final_n;    // [B + P + 2] what k_slab_place needs of the counters above, copied by the last workgroup of
                        // k_slab_classify before it puts them back to zero: moved-in entries per bucket, serial
                        // entries per partition, logged losers, displaced owners
  Counters *ctr;
  uint32_t *coarse_cursor;  // the feed's coarse cursors and, for an fp32 top-k, the refinement histogram (else
  uint32_t *refine_hist;    // null): k_slab_sort puts them back to zero
  int partitions;
  uint32_t log_cap;
};

// The counters and histograms that must be zero when a call starts live in memory that is zero between calls
// (the part of the caller's table the hash map does not use), and every one of them is put back to zero by the
// last kernel that needs it: no kernel spends its time clearing them up front.

// Every kSlabIndexStep-th narrow key range of a bucket (zen_slab.h; about one record per range) has its first
// sorted place written down by the sort kernel: whoever asks who owns a level-1 slot reads two of these places
// and the three or four records between them instead of bisecting the whole bucket (thirteen loads, one
// after the other).
constexpr int kSlabIndexStep = 4;
constexpr int kSlabIndexLen = kSlabSubs / kSlabIndexStep + 1;
static_assert(kSlabSubs % kSlabIndexStep == 0 && kSlabCap < 65536, "index layout");

__device__ inline uint32_t level1_slot(const Probe &g, uint32_t t) { return (poly(t) + kSeed1) % g.m; }

// ---------------------------------------------- coarse slabs -> bucket slabs

// The select kernel leaves its candidates in the coarse slabs (zen_slab_feed.h), as (index, value): index 0 is
// dropped there already, what the exact threshold excludes is dropped on the way to the buckets (the threshold
// is known only when the select kernel has ended).  An entry's level-1 slot is hashed again wherever it is
// needed, which is cheaper than carrying it along.
template <typename S>
struct EncodeSink {
  SlabGeom geo;
  uint32_t *raw_idx;
  S *raw_val;
  const uint32_t *filter;  // optional exact threshold
  __device__ inline bool keep(const uint32_t (&w)[2]) const {
    return (w[1] & KeyOf<S>::kMask) >= (filter ? filter[0] : 0u);
  }
  __device__ inline uint32_t bucket(const uint32_t (&w)[2]) const {
    return geo.bucket_of(geo.mod_m(poly(w[0]) + kSeed1));
  }
  __device__ inline void store(size_t at, const uint32_t (&w)[2]) const {
    raw_idx[at] = w[0];
    raw_val[at] = (S)w[1];
  }
};

// ------------------------------------------------------------ sort a bucket

// Twice the threads of the other per-bucket kernels, half the records each: the phases of this kernel are
// chains of LDS round trips, and eight waves per SIMD hide them better than four (38 -> 30 us); it needs
// fewer than 64 registers, so two workgroups still share a compute unit.
constexpr int kSortBlock = 1024;
constexpr int kSortItems = kSlabCap / kSortBlock;

template <typename S>
__global__ __launch_bounds__(kSortBlock, 8) void k_slab_sort(SlabGeom geo, SlabTables tb, int32_t *status) {
  // the ties take the place of the counters once the ranks are known: with 32-bit values the kernel would
  // otherwise need 88 KB of LDS, one workgroup to a compute unit instead of two
  __shared__ SlabSortSharedNoQueue sh;
  __shared__ S s_val[kSlabCap];
  __shared__ uint32_t s_lost, s_base;
  const uint32_t b = blockIdx.x;
  const size_t base = (size_t)b * kSlabCap;
  uint32_t n_raw = tb.cursor[b * kCursorPad];
  if (n_raw > (uint32_t)kSlabCap) n_raw = kSlabCap;  // the scatter flagged the overflow
  const uint32_t lo = tb.bucket_lo[b];
  S *slab_val = static_cast<S *>(tb.slab_val);
  if (threadIdx.x == 0) s_lost = 0;
  // the kernels before this one were the last to need these: back to zero, a slice per workgroup
  for (uint32_t i = b * kSortBlock + threadIdx.x; i < kCoarseCursorWords; i += gridDim.x * kSortBlock)
    tb.coarse_cursor[i] = 0;
  if (tb.refine_hist)
    for (uint32_t i = b * kSortBlock + threadIdx.x; i <= (uint32_t)kRefineBins; i += gridDim.x * kSortBlock)
      tb.refine_hist[i] = 0;
  uint32_t off[kSortItems], idx[kSortItems], pos[kSortItems], rank[kSortItems];
  S val[kSortItems];
  uint32_t live = 0;
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t j = threadIdx.x + i * kSortBlock;
    // no branch around the loads (places past the end are pulled back onto the slab's first record): they are
    // all in flight together
    const size_t from = base + (j < n_raw ? j : 0u);
    idx[i] = tb.raw_idx[from];
    val[i] = static_cast<const S *>(tb.raw_val)[from];
    off[i] = pos[i] = 0;
    if (j < n_raw) {
      off[i] = geo.mod_m(poly(idx[i]) + kSeed1) - lo;  // the level-1 slot again: cheaper than carrying it along
      pos[i] = j;
      live |= 1u << i;
    }
  }
  // ties between equal slots are broken by the record's place in the slab (13 bits, so a record is one word
  // while it is ranked); the runs of equal slots, few and short, are put right afterwards
  static_assert(kSlabCap <= (1 << 13), "slab places in 13 bits");
  uint32_t n = 0;
  if (!slab_rank<kSortBlock>(sh, geo, 13, off, pos, live, rank, &n)) {
    if (threadIdx.x == 0) {
      tb.cursor[b * kCursorPad] = 0;
      atomicOr(status, ZEN_STAT_RETRY);
      tb.bucket_n[b] = 0;
      tb.removed_n[b] = 0;
    }
    return;
  }
  // every thread has read the slab's fill count (slab_rank synchronised); this workgroup was its only reader
  if (threadIdx.x == 0) tb.cursor[b * kCursorPad] = 0;
  // the counters hold where every narrow range starts in the sorted bucket: every kSlabIndexStep-th goes to
  // the index (before the counters' memory is used for the ties below)
  for (int j = threadIdx.x; j < kSlabIndexLen; j += kSortBlock)
    tb.sub_index[(size_t)b * kSlabIndexLen + j] = (uint16_t)sh.cnt[sub_place<kSortBlock>((uint32_t)j * kSlabIndexStep)];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    if (live & (1u << i)) {
      sh.key[rank[i]] = off[i];
      sh.tie[rank[i]] = idx[i];
      s_val[rank[i]] = val[i];
    }
  }
  __syncthreads();
  // a run of equal slots gets its smallest index in front (the thread at the run's first place does it)
  for (uint32_t p = threadIdx.x; p + 1 < n; p += kSortBlock) {
    const uint32_t k = sh.key[p];
    if (sh.key[p + 1] == k && (p == 0 || sh.key[p - 1] != k)) {
      uint32_t best = p;
      for (uint32_t u = p + 1; u < n && sh.key[u] == k; ++u)
        if (sh.tie[u] < sh.tie[best]) best = u;
      if (best != p) {
        const uint32_t ti = sh.tie[p];
        const S tv = s_val[p];
        sh.tie[p] = sh.tie[best];
        s_val[p] = s_val[best];
        sh.tie[best] = ti;
        s_val[best] = tv;
      }
    }
  }
  __syncthreads();
  // In a run of equal slots the first entry has the smallest index: the slot's level-1 owner.  The others
  // lost level 1.  Their places in the sorted slab are collected where the slots were, once every thread has
  // looked at those (a bucket has at most kSlabSubs of them, else the call is declined).
  uint32_t lost_mask = 0;
#pragma unroll 1
  for (int i = 0; i < kSortItems; ++i) {
    const uint32_t p = threadIdx.x + (uint32_t)i * kSortBlock;
    if (p < n) {
      const uint32_t k = sh.key[p];
      const bool lost = p > 0 && sh.key[p - 1] == k;
      tb.slab_idx[base + p] = (int32_t)(sh.tie[p] | (lost ? kRemovedBit : 0u));
      slab_val[base + p] = s_val[p];  // every thread has read its records: in place is safe
      lost_mask |= lost ? 1u << i : 0u;
    }
  }
  __syncthreads();
#pragma unroll 1
  for (int i = 0; i < kSortItems; ++i) {
    if (lost_mask & (1u << i)) {
      const uint32_t at = atomicAdd(&s_lost, 1u);
      if (at < (uint32_t)kSlabSubs) sh.key[at] = threadIdx.x + (uint32_t)i * kSortBlock;
    }
  }
  __syncthreads();
  uint32_t lost_n = s_lost;
  if (lost_n > (uint32_t)kSlabSubs) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    lost_n = kSlabSubs;
  }
  if (threadIdx.x == 0) {
    tb.bucket_n[b] = n;
    tb.removed_n[b] = lost_n;
    s_base = lost_n ? atomicAdd(&tb.ctr->losers, lost_n) : 0u;
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < lost_n; i += kSortBlock) {
    const uint32_t at = s_base + i;
    const uint32_t p = sh.key[i];
    if (at < tb.log_cap) {
      tb.log_t[at] = sh.tie[p];
      tb.log_v[at] = (uint32_t)s_val[p];
    } else {
      atomicOr(status, ZEN_STAT_RETRY);
    }
  }
}

// ------------------------------------------------------ levels 2 and 3

// Smallest index whose level-1 slot is `slot` (kNone if nobody's), and where it sits.  The bucket's index
// narrows the search to the records of kSlabIndexStep narrow ranges (three or four); they are fetched four at
// a time and looked at in sorted order: by ascending slot, and in a run of equal slots the smallest index
// comes first.
__device__ inline uint32_t slab_head(const SlabGeom &geo, const SlabTables &tb, uint32_t slot, size_t *pos_out,
                                     uint32_t *bucket_out) {
  const uint32_t b = geo.bucket_of(slot);
  const int32_t *idx = tb.slab_idx + (size_t)b * kSlabCap;
  const uint32_t n = tb.bucket_n[b];
  const uint32_t j = ((slot - tb.bucket_lo[b]) >> geo.sub_shift) / (uint32_t)kSlabIndexStep;
  const uint16_t *index = tb.sub_index + (size_t)b * kSlabIndexLen;
  uint32_t p = index[j], end = index[j + 1];
  if (end > n) end = n;  // a bucket the sort declined has no index (and no records)
  for (; p < end; p += 4) {
    uint32_t t[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) t[q] = (uint32_t)idx[p + q < end ? p + q : p] & kIndexMask;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (p + q >= end) return kNone;
      const uint32_t s1 = geo.mod_m(poly(t[q]) + kSeed1);
      if (s1 > slot) return kNone;
      if (s1 == slot) {
        *pos_out = (size_t)b * kSlabCap + p + q;
        *bucket_out = b;
        return t[q];
      }
    }
  }
  return kNone;
}

template <typename S>
__global__ __launch_bounds__(256) void k_slab_chains(SlabGeom geo, Probe g, SlabTables tb, unsigned long long *cells,
                                                     uint32_t log2, int32_t *status) {
  Counters *ctr = tb.ctr;
  uint32_t losers = ctr->losers;
  if (losers > tb.log_cap) losers = tb.log_cap;
  const S *slab_val = static_cast<const S *>(tb.slab_val);
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < losers; i += gridDim.x * 256u) {
    uint32_t cur = tb.log_t[i];
    int lv = 1;
    bool full = false;
    for (uint32_t steps = 0; lv < g.levels; ++steps) {
      if (steps > kChainLimit) {
        atomicOr(status, ZEN_STAT_INTERNAL);
        break;
      }
      uint32_t part;
      const uint32_t slot = probe_slot(g, cur, lv, &part);
      size_t head_pos = 0;
      uint32_t head_bucket = 0;
      const uint32_t head = slab_head(geo, tb, slot, &head_pos, &head_bucket);
      if (head < cur) {  // a smaller index probes this slot at level 1: cur moves on
        ++lv;
        continue;
      }
      const uint32_t old = map_min(cells, log2, slot, cur, ctr, &full);
      if (full) {
        atomicOr(status, ZEN_STAT_RETRY);
        break;
      }
      if (old < cur) {  // a smaller index got here at level 2 or 3
        ++lv;
        continue;
      }
      if (old == kNone) {
        // first level-2/3 prober of this slot: its level-1 owner (a larger index, if any) is pushed out
        if (head == kNone) break;
        atomicOr(reinterpret_cast<uint32_t *>(&tb.slab_idx[head_pos]), kRemovedBit);
        atomicAdd(&tb.removed_n[head_bucket], 1u);
        const uint32_t at = losers + atomicAdd(&ctr->displaced, 1u);
        if (at < tb.log_cap) {
          tb.log_t[at] = head;
          tb.log_v[at] = (uint32_t)slab_val[head_pos];
        } else {
          atomicOr(status, ZEN_STAT_RETRY);
        }
        cur = head;
        lv = 1;
        continue;
      }
      if (old == cur) break;
      // took the slot from a larger index that held it at its first level mapping here
      int lw = 1;
      while (lw < g.levels && probe_slot(g, old, lw, &part) != slot) ++lw;
      cur = old;
      lv = lw + 1;
    }
  }
}

// Where every bucket starts in the output: survivors + moved-in entries, the partition's serial entries
// behind its last bucket.  Run by one workgroup of kSlabBlock threads once all counts are final: it is the last
// to need the counters the chains and the classification raised with atomics, hands what k_slab_place still
// wants of them on in final_n and puts them back to zero.
__device__ inline void slab_output_starts(const SlabGeom &geo, const SlabTables &tb, uint32_t *s_scan) {
  constexpr int kPer = kSlabMaxBuckets / kSlabBlock;
  const uint32_t B = geo.nbuckets;
  uint32_t c[kPer];
  uint32_t sum = 0;
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const uint32_t x = threadIdx.x * kPer + e;
    c[e] = 0;
    if (x < B) {
      const uint32_t mv_raw = load_fresh(&tb.movein_n[x]);
      const uint32_t mv = mv_raw > (uint32_t)kSlabMoveCap ? (uint32_t)kSlabMoveCap : mv_raw;
      tb.final_n[x] = mv_raw;
      tb.movein_n[x] = 0;
      c[e] = tb.bucket_n[x] - load_fresh(&tb.removed_n[x]) + mv;
      if (x % geo.bpp == geo.bpp - 1) {
        const uint32_t sn_raw = load_fresh(&tb.serial_n[x / geo.bpp]);
        tb.final_n[B + x / geo.bpp] = sn_raw;
        tb.serial_n[x / geo.bpp] = 0;
        c[e] += sn_raw > (uint32_t)kSlabSerialCap ? (uint32_t)kSlabSerialCap : sn_raw;
      }
    }
    sum += c[e];
  }
  uint32_t total;
  uint32_t running = block_exclusive_scan<uint32_t, kSlabBlock>(sum, s_scan, &total);
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const uint32_t x = threadIdx.x * kPer + e;
    if (x <= B) tb.out_start[x] = running;
    running += c[e];
  }
  if (B == (uint32_t)kSlabMaxBuckets && threadIdx.x == kSlabBlock - 1) tb.out_start[B] = running;
  if (threadIdx.x == 0) {
    const uint32_t P = (uint32_t)tb.partitions;
    tb.final_n[B + P] = load_fresh(&tb.ctr->losers);
    tb.final_n[B + P + 1] = load_fresh(&tb.ctr->displaced);
    tb.ctr->logged = tb.ctr->losers = tb.ctr->claims = tb.ctr->displaced = 0;
    *tb.done = 0;
  }
}

// Final place of every logged entry: the level-2/3 slot it holds in the map, or its partition's serial list.
// The workgroup that finishes last then knows every count and lays out the output.
__global__ __launch_bounds__(kSlabBlock) void k_slab_classify(SlabGeom geo, Probe g, SlabTables tb,
                                                              const unsigned long long *__restrict__ cells,
                                                              uint32_t log2, int64_t spp, int32_t *status) {
  __shared__ uint32_t s_scan[kSlabBlock / 64 + 1];
  __shared__ bool s_last;
  const Counters *ctr = tb.ctr;
  uint32_t losers = ctr->losers;
  if (losers > tb.log_cap) losers = tb.log_cap;
  uint32_t total = losers + ctr->displaced;
  if (total > tb.log_cap) total = tb.log_cap;
  for (uint32_t i = blockIdx.x * kSlabBlock + threadIdx.x; i < total; i += gridDim.x * kSlabBlock) {
    const uint32_t t = tb.log_t[i];
    uint32_t part = 0, cell = kNone, slot = kNone;
    for (int lv = 1; lv < g.levels && slot == kNone; ++lv) {
      const uint32_t s = probe_slot(g, t, lv, &part);
      uint32_t at = 0;
      if (map_find(cells, log2, s, &at) == t) {
        slot = s;
        cell = at;
      }
    }
    tb.log_cell[i] = cell;
    if (slot != kNone) {
      const uint32_t b = geo.bucket_of(slot);
      const uint32_t at = atomicAdd(&tb.movein_n[b], 1u);
      if (at < (uint32_t)kSlabMoveCap) {
        const size_t dst = (size_t)b * kSlabMoveCap + at;
        tb.mv_key[dst] = slot;
        tb.mv_idx[dst] = t;
        tb.mv_val[dst] = tb.log_v[i];
      } else {
        atomicOr(status, ZEN_STAT_RETRY);
      }
    } else {
      part = level1_slot(g, t) / g.npp;
      const uint32_t at = atomicAdd(&tb.serial_n[part], 1u);
      if (at < (uint32_t)kSlabSerialCap)
        tb.ser_idx[(size_t)part * kSlabSerialCap + at] = t;
      else  // more than the partition's serial region holds is an overflow; more than this path carries, a retry
        atomicOr(status, (int64_t)at >= spp ? ZEN_STAT_SERIAL_OVERFLOW : ZEN_STAT_RETRY);
    }
  }
  // the counters above were raised with atomics that returned (movein_n, serial_n): they have been carried out
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(tb.done, 1u) == gridDim.x - 1u;
  __syncthreads();
  if (s_last) slab_output_starts(geo, tb, s_scan);
}

// ------------------------------------------------------------------ place

constexpr int kPlaceRemoved = 1024;  // removed entries per bucket the place kernel keeps track of

// Ranks the n (distinct) words of `a` in LDS: on return a is ascending.  Called by the whole workgroup; n is
// small in practice (a handful), at most kSlabMoveCap.
__device__ inline void sort_small(uint32_t *a, uint32_t n) {
  constexpr int kPer = kSlabMoveCap / kSlabBlock;
  uint32_t x[kPer], r[kPer];
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const uint32_t j = threadIdx.x + e * kSlabBlock;
    x[e] = j < n ? a[j] : 0u;
    r[e] = 0;
    if (j < n)
      for (uint32_t u = 0; u < n; ++u) r[e] += a[u] < x[e];
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kPer; ++e)
    if (threadIdx.x + e * kSlabBlock < n) a[r[e]] = x[e];
  __syncthreads();
}

// The sorted slab of a bucket is almost its part of the output already: the entries that lost their slot
// (a handful) drop out and the entries that moved in from elsewhere (another handful) slip in between.  So
// an entry at sorted place p goes to
//     bucket start + p - (removed entries before p) + (moved-in entries whose slot is smaller),
// both counts being searches in two short sorted lists; consecutive lanes read consecutive entries and write
// (almost) consecutive places, and nothing but the bucket's slots passes through LDS.
template <typename S>
__global__ __launch_bounds__(kSlabBlock) void k_slab_place(SlabGeom geo, SlabTables tb, unsigned long long *cells,
                                                           int partitions, int64_t spp,
                                                           const S *__restrict__ dense, int32_t *__restrict__ out_idx,
                                                           S *__restrict__ out_val, uint32_t capacity,
                                                           int64_t *__restrict__ splits, int32_t *status) {
  __shared__ uint32_t s_key[kSlabCap];                 // sorted slots of the bucket
  __shared__ uint32_t s_mk[kSlabMoveCap];              // slots of the moved-in entries, ascending
  __shared__ uint32_t s_mp[kSlabMoveCap];              // sorted place in front of which each of them slips in
  __shared__ uint32_t s_rm[kPlaceRemoved];             // sorted places of the removed entries, ascending
  __shared__ int32_t s_delta[kSlabCap / 64];           // per 64 sorted places: how far their entries move
  __shared__ uint32_t s_nrm;
  constexpr int32_t kNoDelta = INT32_MIN;              // the stretch has no common amount
  const uint32_t b = blockIdx.x;
  const uint32_t B = geo.nbuckets;
  const size_t base = (size_t)b * kSlabCap;
  const S *slab_val = static_cast<const S *>(tb.slab_val);
  if (threadIdx.x == 0) s_nrm = 0;

  // every occupied map cell ends with the index that finally holds its slot, and that index recorded the
  // cell: clearing by cell number leaves the borrowed memory zero again
  const uint32_t *serial_n = tb.final_n + B;
  {
    uint32_t losers = tb.final_n[B + tb.partitions];
    if (losers > tb.log_cap) losers = tb.log_cap;
    uint32_t total = losers + tb.final_n[B + tb.partitions + 1];
    if (total > tb.log_cap) total = tb.log_cap;
    for (uint32_t i = b * kSlabBlock + threadIdx.x; i < total; i += B * kSlabBlock) {
      const uint32_t cell = tb.log_cell[i];
      if (cell != kNone) cells[cell] = 0ull;
    }
  }

  const uint32_t n = tb.bucket_n[b];
  uint32_t mv_n = tb.final_n[b];
  if (mv_n > (uint32_t)kSlabMoveCap) mv_n = kSlabMoveCap;
  // the thread's entries (sorted places threadIdx.x + i * kSlabBlock) stay in registers; the slots go to LDS
  // for the searches, the places of removed entries are collected
  uint32_t idx[kSlabItems];
  S val[kSlabItems];
#pragma unroll
  for (int i = 0; i < kSlabItems; ++i) {
    const uint32_t p = threadIdx.x + i * kSlabBlock;
    idx[i] = kRemovedBit;
    val[i] = 0;
    if (p < n) {
      idx[i] = (uint32_t)tb.slab_idx[base + p];
      s_key[p] = geo.mod_m(poly(idx[i] & kIndexMask) + kSeed1);
      val[i] = slab_val[base + p];
    }
  }
  for (uint32_t j = threadIdx.x; j < mv_n; j += kSlabBlock) s_mk[j] = tb.mv_key[(size_t)b * kSlabMoveCap + j];
  __syncthreads();  // s_nrm is zero, s_key and s_mk are there
#pragma unroll
  for (int i = 0; i < kSlabItems; ++i) {
    const uint32_t p = threadIdx.x + i * kSlabBlock;
    if (p < n && (idx[i] & kRemovedBit)) {
      const uint32_t at = atomicAdd(&s_nrm, 1u);
      if (at < (uint32_t)kPlaceRemoved) s_rm[at] = p;
    }
  }
  __syncthreads();
  uint32_t rm_n = s_nrm;
  if (rm_n > (uint32_t)kPlaceRemoved) {  // more collisions than this path carries
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    return;
  }
  if (rm_n > 1) sort_small(s_rm, rm_n);
  // moved-in entry j: its slot's rank among the moved-in slots (they are distinct: a slot has one owner), and
  // the sorted place in front of which it slips in
  uint32_t mj[kSlabMoveCap / kSlabBlock], mplace[kSlabMoveCap / kSlabBlock];
#pragma unroll
  for (int e = 0; e < kSlabMoveCap / kSlabBlock; ++e) {
    const uint32_t j = threadIdx.x + e * kSlabBlock;
    mj[e] = mplace[e] = 0;
    if (j < mv_n) {
      const uint32_t k = s_mk[j];
      uint32_t r = 0;
      for (uint32_t u = 0; u < mv_n; ++u) r += s_mk[u] < k;
      mj[e] = r;
      mplace[e] = lower_bound_u32(s_key, n, k);
    }
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kSlabMoveCap / kSlabBlock; ++e)
    if (threadIdx.x + e * kSlabBlock < mv_n) s_mp[mj[e]] = mplace[e];
  __syncthreads();
  const uint32_t out_base = tb.out_start[b];
  const uint32_t out_n = tb.out_start[b + 1] - out_base;
  // Most stretches of 64 consecutive sorted places contain neither a removed entry nor the place where a
  // moved-in entry slips in: all their entries move by the same amount, found once per stretch.
  for (uint32_t c = threadIdx.x; c * 64u < n; c += kSlabBlock) {
    const uint32_t p0 = c * 64u, p1 = p0 + 63u < n ? p0 + 63u : n - 1u;
    uint32_t mv0 = 0, mv1 = 0, r0 = 0, r1 = 0;
    if (mv_n) {
      mv0 = upper_bound_u32(s_mp, mv_n, p0);
      mv1 = upper_bound_u32(s_mp, mv_n, p1);
    }
    if (rm_n) {
      r0 = lower_bound_u32(s_rm, rm_n, p0);
      r1 = lower_bound_u32(s_rm, rm_n, p1);
    }
    s_delta[c] = (mv0 == mv1 && r0 == r1) ? (int32_t)(mv0 - r0) : kNoDelta;
  }
  __syncthreads();
  // survivors
#pragma unroll
  for (int i = 0; i < kSlabItems; ++i) {
    const uint32_t p = threadIdx.x + i * kSlabBlock;
    if (p < n && !(idx[i] & kRemovedBit)) {
      int32_t delta = s_delta[p >> 6];
      if (delta == kNoDelta)
        delta = (int32_t)((mv_n ? upper_bound_u32(s_mp, mv_n, p) : 0u) - (rm_n ? lower_bound_u32(s_rm, rm_n, p) : 0u));
      const uint32_t pos = out_base + p + (uint32_t)delta;
      if (pos < capacity) {
        out_idx[pos] = (int32_t)idx[i];
        out_val[pos] = val[i];
      }
    }
  }
  // moved-in entries
#pragma unroll
  for (int e = 0; e < kSlabMoveCap / kSlabBlock; ++e) {
    const uint32_t j = threadIdx.x + e * kSlabBlock;
    if (j < mv_n) {
      const uint32_t pos = out_base + mplace[e] + mj[e] - (rm_n ? lower_bound_u32(s_rm, rm_n, mplace[e]) : 0u);
      if (pos < capacity) {
        out_idx[pos] = (int32_t)tb.mv_idx[(size_t)b * kSlabMoveCap + j];
        out_val[pos] = (S)tb.mv_val[(size_t)b * kSlabMoveCap + j];
      }
    }
  }
  const uint32_t part = b / geo.bpp;
  const bool last_of_part = b % geo.bpp == geo.bpp - 1;
  uint32_t serial = 0;
  if (last_of_part) {
    serial = serial_n[part];
    if (serial > (uint32_t)kSlabSerialCap) serial = kSlabSerialCap;
  }
  const uint32_t own_n = out_n - serial;  // survivors + moved-in
  if (serial) {
    // the partition's overflow entries in ascending index order (the reference hands its tickets to
    // ascending thread ids, functions_cuda_kernel.cu:107-108), behind everything that found a slot
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < serial; i += kSlabBlock) s_key[i] = tb.ser_idx[(size_t)part * kSlabSerialCap + i];
    __syncthreads();
    sort_network(s_key, serial);
    for (uint32_t i = threadIdx.x; i < serial; i += kSlabBlock) {
      const uint32_t pos = out_base + own_n + i;
      if (pos < capacity) {
        out_idx[pos] = (int32_t)s_key[i];
        out_val[pos] = dense[s_key[i]];
      }
    }
  }
  if (b % geo.bpp == 0 && threadIdx.x == 0) {
    const uint32_t lo = tb.out_start[b], hi = tb.out_start[b + geo.bpp];
    splits[part] = (int64_t)(hi - lo);
    if ((int64_t)serial_n[part] > spp) atomicOr(status, ZEN_STAT_SERIAL_OVERFLOW);
    if (hi > capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  (void)partitions;
}

struct SlabPlan {
  SlabTables tb;
  uint32_t *sample_hist[2];  // sampled floor histogram (+ finished-block count); two sets, so that the sample of
                             // the next call can be taken (zen_load_balance_prepare) while this call still runs
  uint32_t *cand_hist;
  uint32_t *ticket;
  CoarseGeom cg;
  FeedBuffers feed;
  uint32_t *thr;          // [0..1] exact threshold + count, [2..3] sampled floor, [4] candidates above the k-th's bin,
                          // [6..7] sampled floor of the second set
  uint32_t *refine_hist;  // fp32: histogram of the threshold's last 16 bits (+ finished-workgroup count)
  size_t state_bytes;     // of the zero-between-calls memory
  size_t bytes;           // of the workspace
};

// `state` is memory that is zero between calls (see above); everything else comes out of the workspace.
SlabPlan plan_slab(void *workspace, void *state, const SlabGeom &geo, int partitions, int dtype, int64_t list_cap) {
  SlabPlan p;
  const size_t B = geo.nbuckets;
  {
    Carver cv(state);
    p.sample_hist[0] = cv.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
    p.sample_hist[1] = cv.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
    p.cand_hist = cv.take<uint32_t>((size_t)kCandHistWords);
    p.ticket = cv.take<uint32_t>(select_stage_ticket_words());
    p.tb.cursor = cv.take<uint32_t>(B * kCursorPad);
    p.feed.coarse_cursor = cv.take<uint32_t>(feed_coarse_cursor_words());
    p.tb.movein_n = cv.take<uint32_t>(B);
    p.tb.serial_n = cv.take<uint32_t>((size_t)partitions);
    p.tb.ctr = cv.take<Counters>(1);
    p.tb.done = cv.take<uint32_t>(1);
    p.refine_hist = cv.take<uint32_t>(dtype == ZEN_BF16 ? 1 : (size_t)kRefineBins + 1);
    p.state_bytes = cv.used;
  }
  Carver cv(workspace);
  p.thr = cv.take<uint32_t>(16);
  p.cg = coarse_geometry(geo, list_cap);
  p.feed.coarse_words = cv.take<uint32_t>(feed_coarse_words(p.cg, 2));
  p.tb.bucket_lo = cv.take<uint32_t>(B);
  p.feed.cursor = p.tb.cursor;
  p.feed.bucket_lo = p.tb.bucket_lo;
  p.tb.coarse_cursor = p.feed.coarse_cursor;
  p.tb.refine_hist = nullptr;
  p.tb.partitions = partitions;
  p.tb.out_start = cv.take<uint32_t>(B + 1);
  p.tb.final_n = cv.take<uint32_t>(B + (size_t)partitions + 2);
  p.tb.bucket_n = cv.take<uint32_t>(B);
  p.tb.removed_n = cv.take<uint32_t>(B);
  p.tb.raw_idx = cv.take<uint32_t>(B * kSlabCap);
  p.tb.raw_val = cv.take<char>(B * kSlabCap * (dtype == ZEN_BF16 ? 2 : 4));
  p.tb.slab_idx = cv.take<int32_t>(B * kSlabCap);
  p.tb.slab_val = cv.take<char>(B * kSlabCap * (dtype == ZEN_BF16 ? 2 : 4));
  p.tb.sub_index = cv.take<uint16_t>(B * kSlabIndexLen);
  p.tb.mv_key = cv.take<uint32_t>(B * kSlabMoveCap);
  p.tb.mv_idx = cv.take<uint32_t>(B * kSlabMoveCap);
  p.tb.mv_val = cv.take<uint32_t>(B * kSlabMoveCap);
  p.tb.ser_idx = cv.take<uint32_t>((size_t)partitions * kSlabSerialCap);
  p.tb.log_cap = (uint32_t)(list_cap / 4 + 1024);
  p.tb.log_t = cv.take<uint32_t>(p.tb.log_cap);
  p.tb.log_v = cv.take<uint32_t>(p.tb.log_cap);
  p.tb.log_cell = cv.take<uint32_t>(p.tb.log_cap);
  p.bytes = cv.used;
  return p;
}

template <typename S>
int slab_launch(const SlabBalanceArgs &a, const SlabGeom &geo, const SlabPlan &p, hipStream_t s) {
  const uint32_t B = geo.nbuckets;
  const uint32_t *filter = a.k > 0 ? p.thr : nullptr;
  const S *dense = static_cast<const S *>(a.input);
  {
    ProfScope prof(kProfFeed, s);
    const EncodeSink<S> sink{geo, p.tb.raw_idx, static_cast<S *>(p.tb.raw_val), filter};
    // the select kernel's candidate histogram and ticket counters lie side by side: back to zero here
    const int rc = feed_fine<2, S>(geo, p.cg, sink, p.feed, a.status, s, p.cand_hist,
                                   (uint32_t)(reinterpret_cast<char *>(p.tb.cursor) - reinterpret_cast<char *>(p.cand_hist)) / 4u);
    if (rc != ZEN_OK) return rc;
  }
  {
    ProfScope prof(kProfSlabSort, s);
    k_slab_sort<S><<<dim3(B), dim3(kSortBlock), 0, s>>>(geo, p.tb, a.status);
    ZEN_LAUNCH_CHECK("k_slab_sort");
  }
  {
    ProfScope prof(kProfSlabChains, s);
    k_slab_chains<S><<<dim3(256), dim3(256), 0, s>>>(geo, a.g, p.tb, a.hash, a.hash_log2, a.status);
    ZEN_LAUNCH_CHECK("k_slab_chains");
    k_slab_classify<<<dim3(128), dim3(kSlabBlock), 0, s>>>(geo, a.g, p.tb, a.hash, a.hash_log2, a.spp, a.status);
    ZEN_LAUNCH_CHECK("k_slab_classify");
  }
  {
    ProfScope prof(kProfSlabPlace, s);
    k_slab_place<S><<<dim3(B), dim3(kSlabBlock), 0, s>>>(geo, p.tb, a.hash, a.partitions, a.spp, dense, a.out_idx,
                                                         static_cast<S *>(a.out_val), (uint32_t)a.capacity, a.splits,
                                                         a.status);
    ZEN_LAUNCH_CHECK("k_slab_place");
  }
  return ZEN_OK;
}

}  // namespace

size_t slab_balance_bytes(int64_t m, int partitions, int dtype, int64_t capacity) {
  SlabGeom geo;
  if (!slab_geometry(m, partitions, capacity, kSlabTarget, &geo)) return 0;
  return plan_slab(nullptr, nullptr, geo, partitions, dtype, list_capacity(capacity)).bytes;
}

// The hash map takes the first 8 << hash_log2 bytes of the caller's table (at most half of it: zen_load_balance
// sizes the map so); the counters sit behind it.
size_t slab_state_offset(uint32_t hash_log2) { return align_up((size_t)8 << hash_log2, 256); }

bool slab_balance_fits(int64_t n, int64_t m, int partitions, int dtype, int64_t capacity, int64_t k, SlabGeom *geo) {
  (void)n;
  (void)k;
  if (capacity > 0x1fffffffll) return false;
  SlabGeom g;
  if (!slab_geometry(m, partitions, capacity, kSlabTarget, &g)) return false;
  // slab_geometry wants m >= 2^22: a table of 16 MB or more, of which the map takes at most half and the
  // counters less than 1 MB
  if (geo) *geo = g;
  return true;
}

// The sample of a coming call, or the clearing of one nobody will pick up.  The sampling memory and the floor
// sit at the head of the zero-between-calls memory and of the workspace whatever the geometry and the path.
int slab_prepare(const SlabBalanceArgs &a, hipStream_t s) {
  char *state = reinterpret_cast<char *>(a.hash) + slab_state_offset(a.hash_log2);
  Carver cs(state);
  uint32_t *sample_hist[2];
  sample_hist[0] = cs.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
  sample_hist[1] = cs.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
  Carver cw(a.workspace);
  uint32_t *thr = cw.take<uint32_t>(16);
  const int set = (a.prepared == 2 || a.second) ? 1 : 0;
  uint32_t *floor = thr + 2 + 4 * set;
  if (a.discard) {  // a sample nobody will pick up: its histogram goes back to zero
    launch_fill<uint32_t>(sample_hist[set], 0u, sampled_floor_zero_bytes() / sizeof(uint32_t), s);
    ZEN_LAUNCH_CHECK("slab: discard a sample");
    return ZEN_OK;
  }
  // the sample alone: the floor stays in the workspace until the call proper picks it up
  if (a.k > 0) return topk_sampled_floor(a.input, a.dtype, a.n, a.k, floor, sample_hist[set], s, true);
  return ZEN_OK;
}

int slab_load_balance(const SlabBalanceArgs &a, hipStream_t s) {
  SlabGeom geo;
  if (!slab_balance_fits(a.n, a.g.m, a.partitions, a.dtype, a.capacity, a.k, &geo))
    return fail(ZEN_EINVAL, "slab_load_balance: sizes do not suit the slab layout");
  char *state = reinterpret_cast<char *>(a.hash) + slab_state_offset(a.hash_log2);
  SlabPlan p = plan_slab(a.workspace, state, geo, a.partitions, a.dtype, list_capacity(a.capacity));
  if (slab_state_offset(a.hash_log2) + p.state_bytes > (size_t)a.g.m * sizeof(int32_t))
    return fail(ZEN_EINVAL, "slab_load_balance: table too small for the counters");
  const bool refine = a.k > 0 && a.dtype == ZEN_F32;
  if (refine) p.tb.refine_hist = p.refine_hist;
  StageArgs sc;
  sc.in = a.input;
  sc.dtype = a.dtype;
  sc.n = a.n;
  sc.thr = a.thr;
  sc.geo = geo;
  sc.cg = p.cg;
  sc.coarse_cursor = p.feed.coarse_cursor;
  sc.coarse_words = p.feed.coarse_words;
  sc.ticket = p.ticket;
  sc.status = a.status;
  int rc;
  const int set = (a.prepared == 2 || a.second) ? 1 : 0;
  uint32_t *floor = p.thr + 2 + 4 * set;
  if (a.only_prepare) return slab_prepare(a, s);
  if (a.k > 0) {
    // one pass: everything at or above a floor estimated from a sample goes to the slabs, the exact
    // threshold is read off the candidates' histogram and applied when the buckets are sorted
    if (a.near_key) {
      // the caller knows about where the threshold lies (an earlier call's): everything from 4/128 of a power
      // of two below that key is a candidate, no sample
      sc.thr = a.near_key;
      sc.floor_margin = a.dtype == ZEN_BF16 ? 4u : 4u << 16;
    } else {
      if (!a.prepared &&
          (rc = topk_sampled_floor(a.input, a.dtype, a.n, a.k, floor, p.sample_hist[set], s, true)) != ZEN_OK)
        return rc;
      sc.thr = floor;
    }
    sc.cand_hist = p.cand_hist;
    sc.pick_k = a.k;
    sc.pick_thr = p.thr;
    sc.pick_above = p.thr + 4;
    sc.thr_copy = refine ? nullptr : a.thr_out;  // fp32: the threshold is not final yet
    sc.clear = p.sample_hist[set];  // the sample kernel is through with its histogram
    sc.clear_words = (uint32_t)(sampled_floor_zero_bytes() / sizeof(uint32_t));
  }
  if (a.next_input && a.next_k > 0) {
    sc.next_in = a.next_input;
    sc.next_k = a.next_k;
    sc.next_n = a.next_n;
    sc.next_hist = p.sample_hist[1 - set];
    if (a.next_state) {  // the sampling memory sits at the head of that table's zero-between-calls memory
      Carver cn(a.next_state);
      uint32_t *first = cn.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
      uint32_t *second = cn.take<uint32_t>(sampled_floor_zero_bytes() / sizeof(uint32_t));
      sc.next_hist = set ? first : second;
    }
    sc.next_floor = p.thr + 2 + 4 * (1 - set);
  }
  if ((rc = select_stage_slabs(sc, s)) != ZEN_OK) return rc;
  if (refine) {
    const uint32_t refine_parts = p.cg.groups * (uint32_t)kCoarseSplit;
    k_refine_threshold<<<dim3(refine_parts < 128u ? refine_parts : 128u), dim3(kRefineBlock), 0, s>>>(
        p.cg, 1, p.feed.coarse_cursor, p.feed.coarse_words, static_cast<const uint32_t *>(a.input), p.thr,
        p.thr + 4, (uint32_t)a.k, p.refine_hist, a.thr_out, a.status);
    ZEN_LAUNCH_CHECK("k_refine_threshold");
  }
  if (a.dtype == ZEN_BF16) return slab_launch<uint16_t>(a, geo, p, s);
  return slab_launch<uint32_t>(a, geo, p, s);
}

}  // namespace zen
