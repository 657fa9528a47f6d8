// Receive side: merge many (index, value) payloads.  The reference builds a
// dense zero tensor of the full gradient length, scatter-adds every payload
// into it and extracts the nonzeros again (comm.py:32-50).  Here the entries
// are stably sorted by index, equal indices are summed in fp32 in arrival order
// (the order a sequential scatter_add_ uses, so the result is reproducible),
// zero sums are dropped and the survivors leave in ascending index order.
#include "zen_common.h"
#include "zen_slab.h"
#include "zen_slab_feed.h"
#include "zen_wide.h"

namespace zen {

namespace {

constexpr int kMrgBlock = 512;
constexpr int kMrgItems = 16;  // consecutive sorted entries per thread (few, large tiles: short prefix chain)
constexpr int kMrgTile = kMrgBlock * kMrgItems;

// Validated sort keys.  The payload that travels with a key is the value itself
// (as fp32 bits): the stable sort keeps arrival order, and the reduce kernel
// needs no gather.
template <typename I, typename S>
__global__ __launch_bounds__(256) void k_merge_prep(const I *__restrict__ idx, const S *__restrict__ val, uint32_t r,
                                                    uint32_t dense_n, uint32_t *__restrict__ keys,
                                                    uint32_t *__restrict__ perm, int32_t *status) {
  const uint32_t j = blockIdx.x * 256u + threadIdx.x;
  if (j >= r) return;
  const I k = idx[j];
  const bool ok = k >= 0 && (uint64_t)k < (uint64_t)dense_n;
  if (!ok) atomicOr(status, ZEN_STAT_BAD_INDEX);
  const uint32_t key = ok ? (uint32_t)k : dense_n;  // bad indices sort behind every good one
  keys[j] = key;
  perm[j] = __float_as_uint(KeyOf<S>::to_f32(val[j]));
}

// One tile = kMrgTile consecutive sorted entries.  The tile's keys and values
// are first brought into LDS with coalesced loads; each thread then walks
// kMrgItems consecutive entries in LDS.  A run that continues past the tile is finished from global
// memory by the thread that owns its head.
__device__ inline int mrg_slot(int i) { return i + (i >> 4); }  // one pad word per 16: conflict-free strides

template <typename I>
__global__ __launch_bounds__(kMrgBlock) void k_merge_reduce(
    const uint32_t *__restrict__ keys, const uint32_t *__restrict__ perm, uint32_t r,
    uint32_t dense_n, I *__restrict__ out_idx, float *__restrict__ out_val, int64_t capacity,
    ScanState st, int ntiles, int64_t *out_count, int32_t *status) {
  __shared__ uint32_t s_scan[kMrgBlock / 64 + 1];
  __shared__ uint64_t s_bcast;
  __shared__ int s_tile;
  __shared__ uint32_t s_key[kMrgTile + kMrgTile / 16];
  __shared__ float s_val[kMrgTile + kMrgTile / 16];
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(st.ticket, 1u);
  __syncthreads();
  const int tile = s_tile;
  if (tile >= ntiles) return;
  const uint32_t tile_base = (uint32_t)tile * kMrgTile;
#pragma unroll
  for (int q = 0; q < kMrgItems; ++q) {
    const int local = q * kMrgBlock + threadIdx.x;
    const uint32_t i = tile_base + local;
    uint32_t k = 0xffffffffu;
    float v = 0.0f;
    if (i < r) {
      k = keys[i];
      v = __uint_as_float(perm[i]);
    }
    s_key[mrg_slot(local)] = k;
    s_val[mrg_slot(local)] = v;
  }
  __syncthreads();
  const int first = threadIdx.x * kMrgItems;
  uint32_t k[kMrgItems];
  float sum[kMrgItems];
  uint32_t keep = 0;
  uint32_t prev = first > 0 ? s_key[mrg_slot(first - 1)] : (tile_base > 0 ? keys[tile_base - 1] : 0xffffffffu);
#pragma unroll
  for (int q = 0; q < kMrgItems; ++q) {
    const int local = first + q;
    k[q] = s_key[mrg_slot(local)];
    const bool head = k[q] < dense_n && ((tile_base + local) == 0 || k[q] != prev);
    prev = k[q];
    sum[q] = 0.0f;
    if (head) {
      float acc = 0.0f;  // the dense tensor starts at +0 (comm.py:35)
      int u = local;
      while (u < kMrgTile && s_key[mrg_slot(u)] == k[q]) acc += s_val[mrg_slot(u++)];
      if (u == kMrgTile)
        for (uint32_t g = tile_base + kMrgTile; g < r && keys[g] == k[q]; ++g)
          acc += __uint_as_float(perm[g]);
      sum[q] = acc;
      if (acc != 0.0f) keep |= 1u << q;  // torch.nonzero keeps NaN, drops +-0
    }
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kMrgBlock>((uint32_t)__popc(keep), s_scan, &total);
  const uint64_t tile_start = lookback_exclusive(st, tile, total, status, &s_bcast);
  if (tile == ntiles - 1 && threadIdx.x == 0) {
    const uint64_t all = tile_start + total;
    *out_count = (int64_t)all;
    if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  // compact the kept entries in LDS (everybody is past reading the staged tile:
  // the scan above synchronised), then write them out with consecutive lanes
  uint32_t li = before;
#pragma unroll
  for (int q = 0; q < kMrgItems; ++q) {
    if (keep & (1u << q)) {
      s_key[li] = k[q];
      s_val[li] = sum[q];
      ++li;
    }
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < total; i += kMrgBlock) {
    const uint64_t pos = tile_start + i;
    if (pos < (uint64_t)capacity) {
      out_idx[pos] = (I)s_key[i];
      out_val[pos] = s_val[i];
    }
  }
}

template <typename S>
__global__ __launch_bounds__(256) void k_scatter_dense(const int32_t *__restrict__ idx, const float *__restrict__ sum,
                                                       const int64_t *count, S *__restrict__ dense, uint32_t dense_n);
// The merged indices come out of workspace memory: after a merge that gave up (ZEN_STAT_INTERNAL, ZEN_STAT_RETRY)
// some of them may never have been written, so none is trusted as an address without a look.
template <>
__global__ __launch_bounds__(256) void k_scatter_dense<uint32_t>(const int32_t *__restrict__ idx,
                                                                 const float *__restrict__ sum,
                                                                 const int64_t *count, uint32_t *__restrict__ dense,
                                                                 uint32_t dense_n) {
  const int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (i < *count && (uint32_t)idx[i] < dense_n) dense[idx[i]] = __float_as_uint(sum[i]);
}
template <>
__global__ __launch_bounds__(256) void k_scatter_dense<uint16_t>(const int32_t *__restrict__ idx,
                                                                 const float *__restrict__ sum,
                                                                 const int64_t *count, uint16_t *__restrict__ dense,
                                                                 uint32_t dense_n) {
  const int64_t i = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (i < *count && (uint32_t)idx[i] < dense_n) dense[idx[i]] = f32_to_bf16_rne(sum[i]);
}

// ---------------------------------------------------------- merge on bucket slabs
//
// The indices a destination receives were assigned to it by a hash, so they spread evenly over [0, dense_n):
// the entries go to bucket slabs by index range (zen_slab_feed.h) as (index, arrival number, value) records,
// and one workgroup per bucket sorts its slab by (index, arrival number) inside LDS (one word per record), sums every run of equal
// indices in arrival order, drops zero sums and writes what is left at the place the buckets before it
// leave off (every bucket publishes how much it keeps and adds up what the earlier ones published).

constexpr int kMergeTarget = 3072;   // records a bucket is sized for: duplicates make the buckets less even
// Twice the threads of the scatter kernels, half the records each: the kernel's phases are chains of LDS round
// trips, which eight waves per SIMD hide better than four, and a thread's records then fit 64 registers, so
// that two workgroups share a compute unit.
constexpr int kMergeBlock = 1024;
constexpr int kMergeRecs = kSlabCap / kMergeBlock;  // slab records per thread
constexpr int kMergeItems = 7;       // sorted records per thread while summing (odd: no LDS bank conflicts)
static_assert(kMergeBlock * kMergeItems >= kSlabCap, "every sorted place needs an owner");

// An entry travels as (index, arrival number, value bits); in the bucket slabs the three sit in arrays of their
// own (the value in its own type: ten bytes per bf16 entry).
template <typename I, typename S>
struct MergeSrc {
  SlabGeom geo;
  const I *idx;
  const S *val;
  uint32_t dense_n;
  int32_t *status;
  // the value is fetched again by arrival number when the entry is written: a workgroup's 4096 arrival numbers
  // are consecutive, so those loads hit the 8 KB it has just read
  using Last = S;
  static constexpr int kStaged = 2;
  __device__ inline uint32_t late(const uint32_t (&w)[3], int) const { return (uint32_t)val[w[1]]; }
  __device__ inline bool load(uint32_t e, uint32_t (&w)[3], uint32_t *bucket) const {
    const I k = idx[e];
    if (k < 0 || (uint64_t)k >= (uint64_t)dense_n) {
      atomicOr(status, ZEN_STAT_BAD_INDEX);  // skipped, like everything behind the good ones in the general path
      return false;
    }
    w[0] = (uint32_t)k;
    w[1] = e;
    w[2] = 0;
    *bucket = geo.bucket_of((uint32_t)k);
    return true;
  }
};
template <typename S>
struct MergeSink {
  SlabGeom geo;
  uint32_t *slab_idx, *slab_arr;
  S *slab_val;
  __device__ inline bool keep(const uint32_t (&)[3]) const { return true; }
  __device__ inline uint32_t bucket(const uint32_t (&w)[3]) const { return geo.bucket_of(w[0]); }
  __device__ inline void store(size_t at, const uint32_t (&w)[3]) const {
    slab_idx[at] = w[0];
    slab_arr[at] = w[1];
    slab_val[at] = (S)w[2];
  }
};

template <typename I, typename S>
__global__ __launch_bounds__(kMergeBlock, 8) void k_merge_bucket(SlabGeom geo, uint32_t *__restrict__ cursor,
                                                             uint32_t *__restrict__ coarse_cursor,
                                                             const uint32_t *__restrict__ bucket_lo,
                                                             const uint32_t *__restrict__ slab_idx,
                                                             const uint32_t *__restrict__ slab_arr,
                                                             const S *__restrict__ slab_val,
                                                             I *__restrict__ out_idx, float *__restrict__ out_val,
                                                             int64_t capacity, ScanState st, int tie_bits,
                                                             int64_t *out_count, int32_t *status) {
  __shared__ SlabSortSharedT<true> sh;  // the values take the counters' place once the ranks are known
  __shared__ uint64_t s_scan64[kMergeBlock / 64 + 1];
  __shared__ int s_tile;
  if (threadIdx.x == 0) s_tile = (int)atomicAdd(st.ticket, 1u);
  __syncthreads();
  const int b = s_tile;  // buckets are taken in order, so every earlier bucket already runs
  const int nb = (int)geo.nbuckets;
  if (b >= nb) return;
  const size_t base = (size_t)b * kSlabCap;
  uint32_t n_raw = cursor[b * kCursorPad];
  if (n_raw > (uint32_t)kSlabCap) n_raw = kSlabCap;  // the scatter flagged the overflow
  const uint32_t lo = bucket_lo[b];
  // The counters of the scatter kernels go back to zero (this workgroup was the only reader of its slab's
  // count; the coarse cursors a slice per workgroup), and the last workgroup to finish clears the prefix
  // state: the memory that must be zero when a call starts is zero again when it ends.
  for (uint32_t i = (uint32_t)b * kMergeBlock + threadIdx.x; i < kCoarseCursorWords; i += (uint32_t)nb * kMergeBlock)
    coarse_cursor[i] = 0;
  uint32_t off[kMergeRecs], arr[kMergeRecs], val[kMergeRecs], rank[kMergeRecs];
  uint32_t live = 0;
  // the loads sit in no branch (places past the end are pulled back onto the slab's first record), so that
  // they are all in flight together
#pragma unroll
  for (int i = 0; i < kMergeRecs; ++i) {
    const uint32_t j = threadIdx.x + i * kMergeBlock;
    const size_t from = base + (j < n_raw ? j : 0u);
    off[i] = slab_idx[from] - lo;
    arr[i] = slab_arr[from];
    val[i] = __float_as_uint(KeyOf<S>::to_f32(slab_val[from]));
    if (j < n_raw) live |= 1u << i;
  }
  uint32_t n = 0;
  const bool ranked = slab_rank<kMergeBlock>(sh, geo, tie_bits, off, arr, live, rank, &n);
  if (threadIdx.x == 0) cursor[b * kCursorPad] = 0;  // every thread has read it: slab_rank synchronised
  if (!ranked) {
    if (threadIdx.x == 0) atomicOr(status, ZEN_STAT_RETRY);
    n = 0;  // the bucket contributes nothing; the prefix protocol still gets its (empty) tile
  } else {
#pragma unroll
    for (int i = 0; i < kMergeRecs; ++i) {
      if (live & (1u << i)) {
        sh.key[rank[i]] = off[i];
        sh.tie[rank[i]] = val[i];  // the arrival numbers have done their work: their place takes the values
      }
    }
  }
  __syncthreads();
  // Thread t owns the sorted places [t * per, (t + 1) * per): as few per thread as cover the bucket (and an odd
  // number, which keeps the lanes of a wave on different LDS banks).  It fetches them all at once and walks
  // through them in registers.  A run of equal indices is summed in arrival order from +0 (like the dense
  // tensor of comm.py:35) and belongs to the thread that holds its last record; where that run began before
  // the thread's first place (rare: runs are short next to `per`, long ones come from payloads that overlap),
  // the part in front is summed first, from the run's head on.
  const uint32_t per = ((n + kMergeBlock - 1) / kMergeBlock) | 1u;  // <= kMergeItems
  const uint32_t first = threadIdx.x * per;
  uint32_t k[kMergeItems];
  float sum[kMergeItems];
  uint32_t keep = 0;
  {
    constexpr uint32_t kNoKey = 0xffffffffu;  // offsets are below the bucket width
    float v[kMergeItems];
#pragma unroll
    for (int q = 0; q < kMergeItems; ++q) {
      const uint32_t p = first + q;
      const bool have = (uint32_t)q < per && p < n;
      const uint32_t from = have ? p : 0u;
      k[q] = sh.key[from];
      v[q] = __uint_as_float(sh.tie[from]);
      if (!have) k[q] = kNoKey;
    }
    const uint32_t before_k = first > 0 && first < n ? sh.key[first - 1] : kNoKey;
    const uint32_t after_k = first + per < n ? sh.key[first + per] : kNoKey;
    float acc = 0.0f;
    if (first < n && before_k == k[0]) {
      // the run began before this thread's places: find its head, sum up to the place in front of `first`
      uint32_t head = first - 1;
      while (head > 0) {
        const uint32_t a0 = sh.key[head - 1];
        const uint32_t a1 = sh.key[head >= 2 ? head - 2 : 0u];
        const uint32_t a2 = sh.key[head >= 3 ? head - 3 : 0u];
        const uint32_t a3 = sh.key[head >= 4 ? head - 4 : 0u];
        if (a0 != before_k) break;
        if (head < 2 || a1 != before_k) { head -= 1; break; }
        if (head < 3 || a2 != before_k) { head -= 2; break; }
        if (head < 4 || a3 != before_k) { head -= 3; break; }
        head -= 4;
      }
      for (uint32_t u = head; u < first; u += 4) {
        const float f0 = __uint_as_float(sh.tie[u]);
        const float f1 = __uint_as_float(sh.tie[u + 1 < first ? u + 1 : u]);
        const float f2 = __uint_as_float(sh.tie[u + 2 < first ? u + 2 : u]);
        const float f3 = __uint_as_float(sh.tie[u + 3 < first ? u + 3 : u]);
        acc += f0;
        if (u + 1 < first) acc += f1;
        if (u + 2 < first) acc += f2;
        if (u + 3 < first) acc += f3;
      }
    }
    uint32_t prev = before_k;
#pragma unroll
    for (int q = 0; q < kMergeItems; ++q) {
      const uint32_t next = q + 1 < kMergeItems ? ((uint32_t)(q + 1) < per ? k[q + 1] : after_k) : after_k;
      if (k[q] != kNoKey) {
        if (k[q] != prev) acc = 0.0f;
        acc += v[q];
        prev = k[q];
        sum[q] = acc;
        if (k[q] != next && acc != 0.0f) keep |= 1u << q;  // torch.nonzero keeps NaN, drops +-0
      } else {
        sum[q] = 0.0f;
      }
    }
  }
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kMergeBlock>((uint32_t)__popc(keep), sh.scan, &total);
  // where this bucket's output starts: the sum of what all earlier buckets keep.  Every thread asks for a
  // few of them (bounded wait), nobody waits for a chain of prefixes; while the answers are on their way the
  // kept entries are gathered in LDS (everybody is past reading the sorted bucket: the scan synchronised).
  if (threadIdx.x == 0) desc_store(&st.desc[b], kDescAggregate | total);
  constexpr int kAsk = kSlabMaxBuckets / kMergeBlock;
  uint64_t d[kAsk];
#pragma unroll
  for (int e = 0; e < kAsk; ++e) {
    const int p = (int)threadIdx.x + e * kMergeBlock;
    d[e] = p < b ? desc_load(&st.desc[p]) : kDescAggregate;
  }
  uint32_t li = before;
#pragma unroll
  for (int q = 0; q < kMergeItems; ++q) {
    if (keep & (1u << q)) {
      sh.key[li] = k[q] + lo;
      sh.tie[li] = __float_as_uint(sum[q]);
      ++li;
    }
  }
  uint64_t mine = 0;
  bool gave_up = false;
#pragma unroll
  for (int e = 0; e < kAsk; ++e) {
    const int p = (int)threadIdx.x + e * kMergeBlock;
    uint32_t spins = 0;
    while ((d[e] >> 62) == 0) {
      if (++spins > kSpinLimit) {
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
      d[e] = desc_load(&st.desc[p]);
    }
    mine += d[e] & kDescValue;
  }
  if (gave_up) atomicOr(status, ZEN_STAT_INTERNAL);
  uint64_t all_before;
  block_exclusive_scan<uint64_t, kMergeBlock>(mine, s_scan64, &all_before);  // its barriers also publish the gathered entries
  const uint64_t tile_start = all_before;
  if (b == nb - 1 && threadIdx.x == 0) {
    const uint64_t all = tile_start + total;
    *out_count = (int64_t)all;
    if (all > (uint64_t)capacity) atomicOr(status, ZEN_STAT_CAPACITY);
  }
  for (uint32_t i = threadIdx.x; i < total; i += kMergeBlock) {
    const uint64_t pos = tile_start + i;
    if (pos < (uint64_t)capacity) {
      out_idx[pos] = (I)sh.key[i];
      out_val[pos] = __uint_as_float(sh.tie[i]);
    }
  }
  // every workgroup has read the descriptors it needs before it gets here
  uint32_t *finished = reinterpret_cast<uint32_t *>(st.desc + nb + 1);
  __syncthreads();
  if (threadIdx.x == 0) s_tile = atomicAdd(finished, 1u) == (uint32_t)nb - 1u;
  __syncthreads();
  if (s_tile) {
    for (int i = threadIdx.x; i < nb; i += kMergeBlock) st.desc[i] = 0ull;
    if (threadIdx.x == 0) {
      *st.ticket = 0;
      *finished = 0;
    }
  }
}

// Memory that must be zero when a merge starts: the prefix state over the buckets and the scatter kernels'
// counters, for the largest geometry.  It sits at the head of the workspace whatever path a call takes, and a
// call on bucket slabs leaves it zero again, so that a caller who vouches for it (ZEN_MODE_ZEROED) saves the
// kernel that would clear it.
constexpr size_t kMergeZeroBytes =
    ((scan_words_c(kSlabMaxBuckets) * sizeof(unsigned long long) + 255) / 256 * 256) +
    (size_t)kCoarseCursorWords * sizeof(uint32_t) + (size_t)kSlabMaxBuckets * kCursorPad * sizeof(uint32_t);

struct SlabMergePlan {
  unsigned long long *scan;  // prefix state over the buckets (zeroed before use)
  CoarseGeom cg;
  FeedBuffers feed;
  uint32_t *slab_idx, *slab_arr;
  void *slab_val;
  size_t zero_bytes;
  size_t bytes;
};

SlabMergePlan plan_slab_merge(void *workspace, const SlabGeom &geo, int64_t r) {  // sized for 4-byte values
  Carver cv(workspace);
  SlabMergePlan p;
  const size_t B = geo.nbuckets;
  p.scan = cv.take<unsigned long long>(scan_words((int64_t)B));
  p.feed.coarse_cursor = cv.take<uint32_t>(feed_coarse_cursor_words());
  p.feed.cursor = cv.take<uint32_t>(B * kCursorPad);
  p.zero_bytes = cv.used;
  cv.used = kMergeZeroBytes;  // whatever the geometry, the rest starts behind the largest zero region
  p.feed.bucket_lo = cv.take<uint32_t>(B);
  p.cg = coarse_geometry(geo, r);
  p.feed.coarse_words = cv.take<uint32_t>(feed_coarse_words(p.cg, 3));
  p.slab_idx = cv.take<uint32_t>(B * kSlabCap);
  p.slab_arr = cv.take<uint32_t>(B * kSlabCap);
  p.slab_val = cv.take<uint32_t>(B * kSlabCap);
  p.bytes = cv.used;
  return p;
}

bool slab_merge_fits(int64_t r, int64_t dense_n, SlabGeom *geo) {
  SlabGeom g;
  if (r < (1 << 15) || r > 0x7ffffffell || !slab_geometry(dense_n, 1, r, kMergeTarget, &g)) return false;
  if (g.sub_shift + ceil_log2_u64((uint64_t)r) > 32) return false;  // (index inside a narrow range, arrival number) must fit a word
  if (geo) *geo = g;
  return true;
}

template <typename I, typename S>
int slab_merge_launch(const SlabGeom &geo, const I *idx, const S *val, int64_t r, int64_t dense_n, void *out_idx,
                      int idx64_out, float *out_val, int64_t capacity, int64_t *out_count, void *workspace,
                      bool zeroed, int32_t *status, hipStream_t s) {
  const SlabMergePlan p = plan_slab_merge(workspace, geo, r);
  if (!zeroed) {
    launch_fill<unsigned long long>(p.scan, 0ull, p.zero_bytes / sizeof(unsigned long long), s);
    ZEN_LAUNCH_CHECK("merge: clear prefix state");
  }
  {
    ProfScope prof(kProfMergeFeed, s);
    const MergeSrc<I, S> src{geo, idx, val, (uint32_t)dense_n, status};
    const MergeSink<S> sink{geo, p.slab_idx, p.slab_arr, static_cast<S *>(p.slab_val)};
    const int rc = feed_slabs<3>(geo, p.cg, src, sink, nullptr, r, p.feed, status, s);
    if (rc != ZEN_OK) return rc;
  }
  const ScanState st = scan_state(p.scan, (int64_t)geo.nbuckets);
  const int tie_bits = ceil_log2_u64((uint64_t)r);  // arrival numbers are < r
  ProfScope prof(kProfMergeBucket, s);
  if (idx64_out)
    k_merge_bucket<int64_t, S><<<dim3(geo.nbuckets), dim3(kMergeBlock), 0, s>>>(
        geo, p.feed.cursor, p.feed.coarse_cursor, p.feed.bucket_lo, p.slab_idx, p.slab_arr,
        static_cast<const S *>(p.slab_val), static_cast<int64_t *>(out_idx), out_val, capacity, st, tie_bits, out_count,
        status);
  else
    k_merge_bucket<int32_t, S><<<dim3(geo.nbuckets), dim3(kMergeBlock), 0, s>>>(
        geo, p.feed.cursor, p.feed.coarse_cursor, p.feed.bucket_lo, p.slab_idx, p.slab_arr,
        static_cast<const S *>(p.slab_val), static_cast<int32_t *>(out_idx), out_val, capacity, st, tie_bits, out_count,
        status);
  ZEN_LAUNCH_CHECK("k_merge_bucket");
  return ZEN_OK;
}

struct MergePlan {
  uint32_t *keys, *tmp_v, *sort_k, *sort_v;
  void *scan;  // prefix state of the reduce kernel
  void *sort_scratch;
  size_t bytes;
  int ntiles;
};

MergePlan plan_merge(void *workspace, int64_t r, int64_t dense_n) {
  Carver cv(workspace);
  cv.used = kMergeZeroBytes;  // the head of the workspace belongs to the bucket-slab path's counters
  MergePlan p;
  const size_t cap = (size_t)(r > 0 ? r : 1);
  p.keys = cv.take<uint32_t>(cap);
  p.tmp_v = cv.take<uint32_t>(cap);
  p.sort_k = cv.take<uint32_t>(cap);
  p.sort_v = cv.take<uint32_t>(cap);
  p.ntiles = (int)ceil_div((int64_t)cap, kMrgTile);
  p.scan = cv.take<unsigned long long>(scan_words(p.ntiles));
  p.sort_scratch = cv.take<char>(sort_scratch_bytes((int64_t)cap));
  p.bytes = cv.used;
  SlabGeom geo;
  if (slab_merge_fits(r, dense_n, &geo)) {
    const size_t slabs = plan_slab_merge(nullptr, geo, r).bytes;
    if (slabs > p.bytes) p.bytes = slabs;
  }
  const size_t wide = wide_merge_bytes(r, dense_n, wide_device_cus());
  if (wide && kMergeZeroBytes + wide > p.bytes) p.bytes = kMergeZeroBytes + wide;
  return p;
}

template <typename S>
int merge_launch(const void *idx, int idx64_in, const S *val, int64_t r, int64_t dense_n, void *out_idx,
                 int idx64_out, float *out_val, int64_t capacity, int64_t *out_count, int mode, void *workspace,
                 int32_t *status, hipStream_t s) {
  const bool zeroed = (mode & ZEN_MODE_ZEROED) != 0;
  const bool slabs_only = (mode & ZEN_MODE_SLABS) != 0;
  mode &= ~(ZEN_MODE_ZEROED | ZEN_MODE_SLABS);
  SlabGeom geo;
  if (mode == ZEN_MODE_FAST && !slabs_only && wide_merge_fits(r, dense_n, wide_device_cus(), nullptr)) {
    // the zero region at the head of the workspace: the prefix state first, the cursors behind it
    Carver cv(workspace);
    unsigned long long *scan = cv.take<unsigned long long>(scan_words((int64_t)kSlabMaxBuckets));
    uint32_t *cursor = cv.take<uint32_t>(feed_coarse_cursor_words());
    if (!zeroed) {
      launch_fill<unsigned long long>(scan, 0ull, kMergeZeroBytes / sizeof(unsigned long long), s);
      ZEN_LAUNCH_CHECK("merge: clear prefix state");
    }
    WideList list;
    if (!wide_merge_list(idx, idx64_in, val, r, dense_n, cursor, static_cast<char *>(workspace) + kMergeZeroBytes,
                         wide_device_cus(), status, &list))
      return fail(ZEN_EINVAL, "zen_merge: sizes do not suit the wide buckets");
    return wide_merge(list, sizeof(S) == 2 ? ZEN_BF16 : ZEN_F32, false, out_idx, idx64_out, out_val, capacity, out_count,
                      scan, s);
  }
  if (mode == ZEN_MODE_FAST && slab_merge_fits(r, dense_n, &geo)) {
    if (idx64_in)
      return slab_merge_launch(geo, static_cast<const int64_t *>(idx), val, r, dense_n, out_idx, idx64_out, out_val,
                               capacity, out_count, workspace, zeroed, status, s);
    return slab_merge_launch(geo, static_cast<const int32_t *>(idx), val, r, dense_n, out_idx, idx64_out, out_val,
                             capacity, out_count, workspace, zeroed, status, s);
  }
  MergePlan p = plan_merge(workspace, r, dense_n);
  const unsigned blocks = (unsigned)ceil_div(r, 256);
  launch_fill<unsigned long long>(static_cast<unsigned long long *>(p.scan), 0ull, scan_words(p.ntiles), s);
  {
    ProfScope prof(kProfMergePrep, s);
    if (idx64_in)
      k_merge_prep<int64_t, S><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const int64_t *>(idx), val, (uint32_t)r,
                                                                  (uint32_t)dense_n, p.keys, p.tmp_v, status);
    else
      k_merge_prep<int32_t, S><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const int32_t *>(idx), val, (uint32_t)r,
                                                                  (uint32_t)dense_n, p.keys, p.tmp_v, status);
    ZEN_LAUNCH_CHECK("k_merge_prep");
  }
  const uint32_t *sk, *sp;
  {
    // fast mode: indices that a hash assigned to one destination spread evenly over the dense length, so
    // the bucket sort applies; a crowded key range makes it raise ZEN_STAT_RETRY
    ProfScope prof(kProfSort, s);
    int where;
    if (mode == ZEN_MODE_FAST && bucket_sort_fits(r, (uint32_t)dense_n))
      where = bucket_sort_pairs(p.keys, p.tmp_v, p.sort_k, p.sort_v, r, nullptr, (uint32_t)dense_n, p.sort_scratch,
                                status, s);
    else
      where = sort_pairs(p.keys, p.tmp_v, p.sort_k, p.sort_v, r, nullptr, ceil_log2_u64((uint64_t)dense_n),
                         p.sort_scratch, status, s);
    if (where < 0) return where;
    sk = where ? p.sort_k : p.keys;
    sp = where ? p.sort_v : p.tmp_v;
  }
  const ScanState st = scan_state(p.scan, p.ntiles);
  ProfScope prof(kProfMergeReduce, s);
  if (idx64_out)
    k_merge_reduce<int64_t><<<dim3((unsigned)p.ntiles), dim3(kMrgBlock), 0, s>>>(
        sk, sp, (uint32_t)r, (uint32_t)dense_n, static_cast<int64_t *>(out_idx), out_val, capacity, st, p.ntiles,
        out_count, status);
  else
    k_merge_reduce<int32_t><<<dim3((unsigned)p.ntiles), dim3(kMrgBlock), 0, s>>>(
        sk, sp, (uint32_t)r, (uint32_t)dense_n, static_cast<int32_t *>(out_idx), out_val, capacity, st, p.ntiles,
        out_count, status);
  ZEN_LAUNCH_CHECK("k_merge_reduce");
  return ZEN_OK;
}

int merge_check(const void *idx, const void *val, int dtype, int64_t r, int64_t dense_n, int mode, const char **why) {
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) { *why = "bad dtype"; return ZEN_EINVAL; }
  if ((mode & ~(ZEN_MODE_ZEROED | ZEN_MODE_SLABS)) != ZEN_MODE_FAST &&
      (mode & ~(ZEN_MODE_ZEROED | ZEN_MODE_SLABS)) != ZEN_MODE_GENERAL) {
    *why = "bad mode";
    return ZEN_EINVAL;
  }
  if (r < 0 || r > 0x7ffffffell || dense_n <= 0 || dense_n > 0x7fffffffll) {
    *why = "need 0 <= r < 2^31 - 1 and 0 < dense_n < 2^31";
    return ZEN_EINVAL;
  }
  if (r > 0 && (!idx || !val)) { *why = "null pointer"; return ZEN_EINVAL; }
  return ZEN_OK;
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_merge_workspace(int64_t r, int64_t dense_n) {
  if (r < 0 || dense_n <= 0) return 0;
  return zen::plan_merge(nullptr, r, dense_n).bytes;
}

size_t zen_merge_zero_bytes(void) { return zen::kMergeZeroBytes; }

int zen_merge_path(int64_t r, int64_t dense_n, int mode) {
  const bool slabs_only = (mode & ZEN_MODE_SLABS) != 0;
  mode &= ~(ZEN_MODE_ZEROED | ZEN_MODE_SLABS);
  if (mode != ZEN_MODE_FAST || r <= 0 || dense_n <= 0) return 0;
  if (!slabs_only && zen::wide_merge_fits(r, dense_n, zen::wide_device_cus(), nullptr)) return 3;
  if (zen::slab_merge_fits(r, dense_n, nullptr)) return 2;
  return zen::bucket_sort_fits(r, (uint32_t)dense_n) ? 1 : 0;
}

int zen_merge(const void *idx, int idx64_in, const void *val, int dtype, int64_t r, int64_t dense_n, void *out_idx,
              int idx64_out, float *out_val, int64_t capacity, int64_t *out_count, int mode, void *workspace,
              size_t workspace_bytes, int32_t *status, void *stream) {
  using namespace zen;
  const char *why = "";
  if (merge_check(idx, val, dtype, r, dense_n, mode, &why) != ZEN_OK) return fail(ZEN_EINVAL, why);
  if (!out_count || !status || capacity < 0) return fail(ZEN_EINVAL, "zen_merge: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (r == 0) {
    launch_fill<int64_t>(out_count, 0, 1, s);
    ZEN_LAUNCH_CHECK("zen_merge: zero count");
    return ZEN_OK;
  }
  if (!workspace || (capacity > 0 && (!out_idx || !out_val))) return fail(ZEN_EINVAL, "zen_merge: null pointer");
  if (workspace_bytes < zen_merge_workspace(r, dense_n)) return fail(ZEN_EWORKSPACE, "zen_merge: workspace too small");
  if (dtype == ZEN_BF16)
    return merge_launch(idx, idx64_in, static_cast<const uint16_t *>(val), r, dense_n, out_idx, idx64_out, out_val,
                        capacity, out_count, mode, workspace, status, s);
  return merge_launch(idx, idx64_in, static_cast<const uint32_t *>(val), r, dense_n, out_idx, idx64_out, out_val,
                      capacity, out_count, mode, workspace, status, s);
}

size_t zen_decode_dense_workspace(int64_t r, int64_t dense_n) {
  if (r < 0 || dense_n <= 0) return 0;
  const size_t cap = (size_t)(r > 0 ? r : 1);
  return zen::align_up(cap * sizeof(int32_t), 256) + zen::align_up(cap * sizeof(float), 256) + 256 +
         zen_merge_workspace(r, dense_n);
}

int zen_decode_dense(const void *idx, int idx64_in, const void *val, int dtype, int64_t r, void *dense,
                     int64_t dense_n, int mode, void *workspace, size_t workspace_bytes, int32_t *status,
                     void *stream) {
  using namespace zen;
  const char *why = "";
  if (merge_check(idx, val, dtype, r, dense_n, mode, &why) != ZEN_OK) return fail(ZEN_EINVAL, why);
  if (!dense || !status) return fail(ZEN_EINVAL, "zen_decode_dense: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == ZEN_BF16)
    launch_fill<uint16_t>(static_cast<uint16_t *>(dense), (uint16_t)0, (size_t)dense_n, s);
  else
    launch_fill<uint32_t>(static_cast<uint32_t *>(dense), 0u, (size_t)dense_n, s);
  ZEN_LAUNCH_CHECK("zen_decode_dense: clear");
  if (r == 0) return ZEN_OK;
  if (!workspace) return fail(ZEN_EINVAL, "zen_decode_dense: null pointer");
  if (workspace_bytes < zen_decode_dense_workspace(r, dense_n))
    return fail(ZEN_EWORKSPACE, "zen_decode_dense: workspace too small");
  Carver cv(workspace);
  int32_t *m_idx = cv.take<int32_t>((size_t)r);
  float *m_val = cv.take<float>((size_t)r);
  int64_t *m_count = cv.take<int64_t>(1);
  void *inner = cv.take<char>(zen_merge_workspace(r, dense_n));
  int rc;
  if (dtype == ZEN_BF16)
    rc = merge_launch(idx, idx64_in, static_cast<const uint16_t *>(val), r, dense_n, m_idx, 0, m_val, r, m_count,
                      mode & ~ZEN_MODE_ZEROED, inner, status, s);
  else
    rc = merge_launch(idx, idx64_in, static_cast<const uint32_t *>(val), r, dense_n, m_idx, 0, m_val, r, m_count,
                      mode & ~ZEN_MODE_ZEROED, inner, status, s);
  if (rc != ZEN_OK) return rc;
  const unsigned blocks = (unsigned)ceil_div(r, 256);
  if (dtype == ZEN_BF16)
    k_scatter_dense<uint16_t><<<dim3(blocks), dim3(256), 0, s>>>(m_idx, m_val, m_count, static_cast<uint16_t *>(dense),
                                                                 (uint32_t)dense_n);
  else
    k_scatter_dense<uint32_t><<<dim3(blocks), dim3(256), 0, s>>>(m_idx, m_val, m_count, static_cast<uint32_t *>(dense),
                                                                 (uint32_t)dense_n);
  ZEN_LAUNCH_CHECK("k_scatter_dense");
  return ZEN_OK;
}

}  // extern "C"

namespace zen {
namespace {

// The merged entries on their way to the second exchange (comm.py:125-127 turns the dense fp32 sums into the
// tensor's type and takes the nonzeros again): every sum is rounded once to the type V, entries whose sum
// rounds to zero are dropped, the others keep their order.  One pass: a tile of kRcBlock * kRcItems entries per
// workgroup, the tiles' kept counts chained by look-back.  count sits on the device.
constexpr int kRcBlock = 256, kRcItems = 8, kRcTile = kRcBlock * kRcItems;
template <typename I, typename V>
__global__ __launch_bounds__(kRcBlock) void k_round_compact(const I *__restrict__ idx, const float *__restrict__ sums,
                                                            const int64_t *__restrict__ count, int64_t capacity,
                                                            I *__restrict__ out_idx, V *__restrict__ out_val,
                                                            int64_t *out_count, ScanState st, int32_t *status) {
  __shared__ uint32_t tile_s;
  __shared__ uint32_t scan_s[kRcBlock / 64 + 1];
  __shared__ uint64_t base_s;
  if (threadIdx.x == 0) tile_s = atomicAdd(st.ticket, 1u);
  __syncthreads();
  const uint32_t tile = tile_s;
  int64_t n = *count;
  if (n > capacity) n = capacity;
  const int64_t first = (int64_t)tile * kRcTile + (int64_t)threadIdx.x * kRcItems;
  I k[kRcItems];
  V v[kRcItems];
  uint32_t keep = 0, mine = 0;
#pragma unroll
  for (int i = 0; i < kRcItems; ++i) {
    const int64_t j = first + i;
    k[i] = 0;
    v[i] = 0;
    if (j < n) {
      k[i] = idx[j];
      const float f = sums[j];
      if constexpr (sizeof(V) == 2) {
        v[i] = f32_to_bf16_rne(f);
        if (v[i] & 0x7fffu) keep |= 1u << i;
      } else {
        v[i] = __float_as_uint(f);
        if (v[i] & 0x7fffffffu) keep |= 1u << i;
      }
    }
  }
  mine = __popc(keep);
  uint32_t total;
  const uint32_t before = block_exclusive_scan<uint32_t, kRcBlock>(mine, scan_s, &total);
  const uint64_t base = lookback_exclusive(st, (int)tile, total, status, &base_s);
  uint64_t at = base + before;
#pragma unroll
  for (int i = 0; i < kRcItems; ++i)
    if (keep & (1u << i)) {
      out_idx[at] = k[i];
      out_val[at] = v[i];
      ++at;
    }
  if (tile == gridDim.x - 1 && threadIdx.x == kRcBlock - 1) *out_count = (int64_t)(base + before + mine);
}

}  // namespace
}  // namespace zen

extern "C" {

size_t zen_round_compact_workspace(int64_t capacity) {
  if (capacity < 0) return 0;
  return zen::scan_words(zen::ceil_div(capacity > 0 ? capacity : 1, (int64_t)zen::kRcTile)) * sizeof(uint64_t);
}

int zen_round_compact(const void *idx, int idx64, const float *sums, const int64_t *count, int64_t capacity, int dtype,
                      void *out_idx, void *out_val, int64_t *out_count, void *workspace, size_t workspace_bytes,
                      int32_t *status, void *stream) {
  using namespace zen;
  if (!count || !out_count || !status || capacity < 0) return fail(ZEN_EINVAL, "zen_round_compact: null pointer");
  if (dtype != ZEN_F32 && dtype != ZEN_BF16) return fail(ZEN_EINVAL, "zen_round_compact: bad dtype");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (capacity == 0) {
    launch_fill<int64_t>(out_count, 0, 1, s);
    ZEN_LAUNCH_CHECK("zen_round_compact: zero count");
    return ZEN_OK;
  }
  if (!idx || !sums || !out_idx || !out_val || !workspace) return fail(ZEN_EINVAL, "zen_round_compact: null pointer");
  if (workspace_bytes < zen_round_compact_workspace(capacity))
    return fail(ZEN_EWORKSPACE, "zen_round_compact: workspace too small");
  const int64_t tiles = ceil_div(capacity, (int64_t)kRcTile);
  if (tiles > 0x7fffffffll) return fail(ZEN_EINVAL, "zen_round_compact: too many entries");
  launch_fill<uint64_t>(static_cast<uint64_t *>(workspace), 0ull, scan_words(tiles), s);
  ZEN_LAUNCH_CHECK("zen_round_compact: clear");
  const ScanState st = scan_state(workspace, tiles);
  const dim3 grid((unsigned)tiles), block(kRcBlock);
#define ZEN_RC(I, V)                                                                                              \
  k_round_compact<I, V><<<grid, block, 0, s>>>(static_cast<const I *>(idx), sums, count, capacity,              \
                                               static_cast<I *>(out_idx), static_cast<V *>(out_val), out_count, \
                                               st, status)
  if (idx64) {
    if (dtype == ZEN_BF16) ZEN_RC(int64_t, uint16_t); else ZEN_RC(int64_t, uint32_t);
  } else {
    if (dtype == ZEN_BF16) ZEN_RC(int32_t, uint16_t); else ZEN_RC(int32_t, uint32_t);
  }
#undef ZEN_RC
  ZEN_LAUNCH_CHECK("k_round_compact");
  return ZEN_OK;
}

}  // extern "C"
